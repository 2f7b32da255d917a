// Merge of the block-major selected-attention partials of one (token, q head, 8 output channels),
// the gates and the sum of the three branches.  Shared by the stand-alone merge kernel and by the
// sliding-window kernel's epilogue.
#pragma once
#include "tiles.h"

namespace nsa {

__device__ __forceinline__ float gate_of(float x, int act) { return act == 1 ? 1.0f / (1.0f + __expf(-x)) : x; }

// slotmap[(tg*hkv + h)*top_n + i] = pair number of pick i, or -1 when the pick is unusable (past
// the count, not a block, beyond the token).  TOPN > 0: the slot map is read with vector loads and
// all partials of the piece are requested before any is used (up to TOPN 16-byte loads in flight
// per lane); TOPN = 0: any top_n, one partial at a time.  n = head inside the GQA group,
// row = token * hq + q head.
// Returns g_slc * o_slc + g_swa * o_swa + g_cmp * o_cmp for the piece (o_swa given by the caller).
template <typename T, int DV, int TOPN, bool EXACT = false>
__device__ __forceinline__ vec8_t<T> merge_piece(const MergeArgs& m, long tg, int h, int n, long row, int pc,
                                                 bool has_swa, const vec8_t<T>& o_swa) {
  const int top_n = EXACT ? TOPN : m.top_n;       // EXACT: top_n == TOPN known at compile time
  const long base = (tg * m.hkv + h) * top_n;
  const float c_attn = m.scale * kLog2e;
  const T* pob = reinterpret_cast<const T*>(m.po);
  float den = 0.f, acc[8], M = kNegInf;
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = 0.f;
  if constexpr (TOPN > 0) {
    // rounds of TOPN picks, exactly as merge_two sums them (the two agree bit for bit)
    const bool quads = top_n % 4 == 0;
    for (int r0 = 0; r0 < top_n; r0 += TOPN) {
      int ps[TOPN];
      if (quads) {
#pragma unroll
        for (int i = 0; i < TOPN / 4; ++i) {
          int4 q4 = {-1, -1, -1, -1};
          if (r0 + 4 * i < top_n) q4 = *reinterpret_cast<const int4*>(m.slotmap + base + r0 + 4 * i);
          ps[4 * i] = q4.x; ps[4 * i + 1] = q4.y; ps[4 * i + 2] = q4.z; ps[4 * i + 3] = q4.w;
        }
      } else {
#pragma unroll
        for (int i = 0; i < TOPN; ++i) ps[i] = r0 + i < top_n ? m.slotmap[base + r0 + i] : -1;
      }
      // all of the slot map before the first partial is requested (the conditional loads below would otherwise be
      // split into batches by a wait for the later parts of the map)
#pragma unroll
      for (int i = 0; i < TOPN; ++i) asm volatile("" ::"v"(ps[i]));
      float mx[TOPN], l[TOPN];
      vec8_t<T> o[TOPN];
#pragma unroll
      for (int i = 0; i < TOPN; ++i) {
        mx[i] = kNegInf; l[i] = 0.f; o[i] = zero8<T>();
        if (ps[i] >= 0) {
          const long p = ps[i];
          mx[i] = m.ml[(p * 2) * 16 + n];
          l[i] = m.ml[(p * 2 + 1) * 16 + n];
          o[i] = load8(pob + (p * m.part_rows + n) * DV + pc * 8);
        }
      }
      float Mr = M;
#pragma unroll
      for (int i = 0; i < TOPN; ++i) Mr = fmaxf(Mr, mx[i]);
      if (r0 > 0 && Mr > M) {
        const float f = fast_exp2((M - Mr) * c_attn);
        den *= f;
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[e] *= f;
      }
      M = Mr;
#pragma unroll
      for (int i = 0; i < TOPN; ++i) {
        if (ps[i] >= 0) {          // the same for every lane that works on this token: unusable picks cost nothing
          const float w = fast_exp2((mx[i] - M) * c_attn) * l[i];
          den += w;
#pragma unroll
          for (int e = 0; e < 8; ++e) acc[e] = fmaf(w, (float)o[i][e], acc[e]);
        }
      }
    }
  } else {
    for (int i = 0; i < top_n; ++i) {
      const long p = m.slotmap[base + i];
      if (p < 0) continue;
      const float mi = m.ml[(p * 2) * 16 + n];
      const float l = m.ml[(p * 2 + 1) * 16 + n];
      const vec8_t<T> o = load8(pob + (p * m.part_rows + n) * DV + pc * 8);
      const float m_new = fmaxf(M, mi);
      const float r_old = fast_exp2((M - m_new) * c_attn);        // 0 for the first partial
      const float w = fast_exp2((mi - m_new) * c_attn) * l;
      den = den * r_old + w;
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[e] = acc[e] * r_old + w * (float)o[e];
      M = m_new;
    }
  }
  const float inv = den > 0.f ? 1.0f / den : 0.f;
  if (m.o_slc_out != nullptr) {
    float os[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) os[e] = acc[e] * inv;
    store8(reinterpret_cast<T*>(m.o_slc_out) + row * DV + pc * 8, pack8<T>(os));
  }
  if (m.o_swa_out != nullptr && has_swa) store8(reinterpret_cast<T*>(m.o_swa_out) + row * DV + pc * 8, o_swa);
  if (m.lse_slc_out != nullptr && pc == 0)
    m.lse_slc_out[row] = den > 0.f ? fmaf(M, m.scale, __logf(den)) : __builtin_huge_valf();
  const T* gs = reinterpret_cast<const T*>(m.g_slc);
  const T* gw = reinterpret_cast<const T*>(m.g_swa);
  const T* gcm = reinterpret_cast<const T*>(m.g_cmp);
  const T* ocm = reinterpret_cast<const T*>(m.o_cmp);
  const float w_slc = (gs ? gate_of((float)gs[row * m.gate_stride], m.gate_act) : 1.f) * inv;
  float out[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) out[e] = acc[e] * w_slc;
  if (has_swa) {
    const float w = gw ? gate_of((float)gw[row * m.gate_stride], m.gate_act) : 1.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) out[e] += w * (float)o_swa[e];
  }
  if (ocm) {
    const float w = gcm ? gate_of((float)gcm[row * m.gate_stride], m.gate_act) : 1.f;
    const vec8_t<T> o = load8(ocm + row * DV + pc * 8);
#pragma unroll
    for (int e = 0; e < 8; ++e) out[e] += w * (float)o[e];
  }
  return pack8<T>(out);
}

// Two pieces (pc_a, pc_b) of one row at once, any top_n: the picks are taken in rounds of up to 16; per round the
// slot map, the maxima and the sums are read once and 2 * 16 partial loads are in flight per lane before the first
// is used (the epilogue that calls this is bound by the latency of those loads, not by their bytes); a round after
// the first joins the running state like one more partial.  TOPN is the round size (16); EXACT: top_n == TOPN is
// known at compile time (one round, no bounds on the slots: the benchmark's shape).
template <typename T, int DV, int TOPN, bool EXACT>
__device__ __forceinline__ void merge_two(const MergeArgs& m, long tg, int h, int n, long row, int pc_a, int pc_b,
                                          const vec8_t<T>& swa_a, const vec8_t<T>& swa_b, vec8_t<T>& res_a,
                                          vec8_t<T>& res_b) {
  static_assert(TOPN > 0 && TOPN % 4 == 0, "unrolled merge only");
  const int top_n = EXACT ? TOPN : m.top_n;
  const long base = (tg * m.hkv + h) * top_n;
  const float c_attn = m.scale * kLog2e;
  const T* pob = reinterpret_cast<const T*>(m.po);
  const bool quads = top_n % 4 == 0;       // then a token's slots are 16-byte aligned
  auto load_slots = [&](int r0, int (&ps)[TOPN]) {
    if (quads) {
#pragma unroll
      for (int i = 0; i < TOPN / 4; ++i) {
        int4 q4 = {-1, -1, -1, -1};
        if (r0 + 4 * i < top_n) q4 = *reinterpret_cast<const int4*>(m.slotmap + base + r0 + 4 * i);
        ps[4 * i] = q4.x; ps[4 * i + 1] = q4.y; ps[4 * i + 2] = q4.z; ps[4 * i + 3] = q4.w;
      }
    } else {
#pragma unroll
      for (int i = 0; i < TOPN; ++i) ps[i] = r0 + i < top_n ? m.slotmap[base + r0 + i] : -1;
    }
  };
  int ps[TOPN];
  load_slots(0, ps);
  // The compressed branch's rows and the three gate logits are requested here, after the slot map and before
  // the wait for it: read where they are used (after the partials are summed) they would cost one more memory
  // round trip per call.  The loads are unconditional so that the compiler can count them and wait for the slot
  // map alone; an absent operand reads the slot map instead and the value is ignored.
  const T* gs = reinterpret_cast<const T*>(m.g_slc);
  const T* gw = reinterpret_cast<const T*>(m.g_swa);
  const T* gcm = reinterpret_cast<const T*>(m.g_cmp);
  const T* ocm = reinterpret_cast<const T*>(m.o_cmp);
  const T* dummy = reinterpret_cast<const T*>(m.slotmap);
  const vec8_t<T> ca = load8(ocm ? ocm + row * DV + pc_a * 8 : dummy);
  const vec8_t<T> cb = load8(ocm ? ocm + row * DV + pc_b * 8 : dummy);
  const T gs_raw = *(gs ? gs + row * m.gate_stride : dummy);
  const T gw_raw = *(gw ? gw + row * m.gate_stride : dummy);
  const T gc_raw = *(gcm ? gcm + row * m.gate_stride : dummy);
  float M = kNegInf, den = 0.f, acc_a[8], acc_b[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) { acc_a[e] = 0.f; acc_b[e] = 0.f; }
  for (int r0 = 0; r0 < top_n; r0 += TOPN) {
    if (r0 > 0) load_slots(r0, ps);
    // All of the slot map before the first partial is requested: the partial loads below are conditional, so the
    // in-order memory counter could otherwise only be waited down to zero when a later part of the map is needed,
    // which would split the loads into batches.
#pragma unroll
    for (int i = 0; i < TOPN; ++i) asm volatile("" ::"v"(ps[i]));
    float mx[TOPN], l[TOPN];
    vec8_t<T> oa[TOPN], ob[TOPN];
#pragma unroll
    for (int i = 0; i < TOPN; ++i) {
      mx[i] = kNegInf; l[i] = 0.f; oa[i] = zero8<T>(); ob[i] = zero8<T>();
      if (ps[i] >= 0) {
        const long p = ps[i];
        mx[i] = m.ml[(p * 2) * 16 + n];
        l[i] = m.ml[(p * 2 + 1) * 16 + n];
        oa[i] = load8(pob + (p * m.part_rows + n) * DV + pc_a * 8);
        ob[i] = load8(pob + (p * m.part_rows + n) * DV + pc_b * 8);
      }
    }
    float Mr = M;
#pragma unroll
    for (int i = 0; i < TOPN; ++i) Mr = fmaxf(Mr, mx[i]);
    if (r0 > 0 && Mr > M) {                  // a later round raised the maximum: rescale what is summed already
      const float f = fast_exp2((M - Mr) * c_attn);
      den *= f;
#pragma unroll
      for (int e = 0; e < 8; ++e) { acc_a[e] *= f; acc_b[e] *= f; }
    }
    M = Mr;
#pragma unroll
    for (int i = 0; i < TOPN; ++i) {
      if (ps[i] >= 0) {
        const float w = fast_exp2((mx[i] - M) * c_attn) * l[i];
        den += w;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          acc_a[e] = fmaf(w, (float)oa[i][e], acc_a[e]);
          acc_b[e] = fmaf(w, (float)ob[i][e], acc_b[e]);
        }
      }
    }
  }
  const float inv = den > 0.f ? 1.0f / den : 0.f;
  if (m.o_slc_out != nullptr) {
    float os[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) os[e] = acc_a[e] * inv;
    store8(reinterpret_cast<T*>(m.o_slc_out) + row * DV + pc_a * 8, pack8<T>(os));
#pragma unroll
    for (int e = 0; e < 8; ++e) os[e] = acc_b[e] * inv;
    store8(reinterpret_cast<T*>(m.o_slc_out) + row * DV + pc_b * 8, pack8<T>(os));
  }
  if (m.o_swa_out != nullptr) {
    store8(reinterpret_cast<T*>(m.o_swa_out) + row * DV + pc_a * 8, swa_a);
    store8(reinterpret_cast<T*>(m.o_swa_out) + row * DV + pc_b * 8, swa_b);
  }
  if (m.lse_slc_out != nullptr && pc_a == 0)
    m.lse_slc_out[row] = den > 0.f ? fmaf(M, m.scale, __logf(den)) : __builtin_huge_valf();
  const float w_slc = (gs ? gate_of((float)gs_raw, m.gate_act) : 1.f) * inv;
  const float w_swa = gw ? gate_of((float)gw_raw, m.gate_act) : 1.f;
  float out_a[8], out_b[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    out_a[e] = acc_a[e] * w_slc;
    out_b[e] = acc_b[e] * w_slc;
    out_a[e] += w_swa * (float)swa_a[e];
    out_b[e] += w_swa * (float)swa_b[e];
  }
  if (ocm) {
    const float w = gcm ? gate_of((float)gc_raw, m.gate_act) : 1.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      out_a[e] += w * (float)ca[e];
      out_b[e] += w * (float)cb[e];
    }
  }
  res_a = pack8<T>(out_a);
  res_b = pack8<T>(out_b);
}

// Log-sum-exp (natural log) of the scaled scores over all usable picks of (token tg, kv head h,
// head n of the group); +inf when the token has no usable pick.
__device__ __forceinline__ float merge_lse(const MergeArgs& m, long tg, int h, int n) {
  const long base = (tg * m.hkv + h) * m.top_n;
  const float c_attn = m.scale * kLog2e;
  float M = kNegInf, den = 0.f;
  for (int i = 0; i < m.top_n; ++i) {
    const long p = m.slotmap[base + i];
    if (p < 0) continue;
    const float mi = m.ml[(p * 2) * 16 + n];
    const float l = m.ml[(p * 2 + 1) * 16 + n];
    const float m_new = fmaxf(M, mi);
    den = den * fast_exp2((M - m_new) * c_attn) + l * fast_exp2((mi - m_new) * c_attn);
    M = m_new;
  }
  return den > 0.f ? fmaf(M, m.scale, __logf(den)) : __builtin_huge_valf();
}

}  // namespace nsa
