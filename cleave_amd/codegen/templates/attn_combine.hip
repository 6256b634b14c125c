// ---- split-KV combine shared by the decode-attention kernels -------------------------------
// Partials are (split, row[, d]) f32 with m the running max in the log2 domain, l the sum of
// weights relative to m, and O the unnormalised weighted values.
#ifndef CL_CHUNK_PAGES
#define CL_CHUNK_PAGES 0
#endif
#ifndef CL_PO_ELEM
#define CL_PO_ELEM 0
#endif
#if CL_CHUNK_PAGES && CL_EMIT_COMBINE
// Combine of chunked items: request b owns items b + p0/C .. b + (p1-1)/C (p0, p1 its page-table
// range); partials are (item, query head[, d]).  One thread per (request, head, 4 d).
extern "C" __global__ void __launch_bounds__(256)
CL_COMBINE_NAME(CL_COMBINE_PARAMS) {
  const i64 total = (i64)CL_TOTAL_ROWS * (CL_VDIM / 4);
  const i64 idx = (i64)blockIdx.x * 256 + threadIdx.x;
  if (idx >= total) return;
  const i64 row = idx / (CL_VDIM / 4);
  const int d = (int)(idx % (CL_VDIM / 4)) * 4;
  const int req = (int)(row / CL_Q_HEADS), qh = (int)(row % CL_Q_HEADS);
  int p0 = CL_CARG_INDPTR[req], p1 = CL_CARG_INDPTR[req + 1];
  p0 = p0 < 0 ? 0 : (p0 > n_idx ? n_idx : p0);
  p1 = p1 < 0 ? 0 : (p1 > n_idx ? n_idx : p1);
  const int first = req + p0 / chunk_pages;
  const int count = p1 > p0 ? (p1 - 1) / chunk_pages - p0 / chunk_pages + 1 : 0;
  // One pass, eight items at a time, every load of a group issued before the first use (the trip
  // count is a run-time value: left alone, each item's loads wait for the previous item's).  The
  // running maximum is carried along and the sums rescaled when a group raises it, so a request of
  // up to eight items costs one round trip to memory; slots past the end repeat the last item with
  // weight zero.
  float m = CL_NEG_BIG, l = 0.f;
  f32x4 o = (f32x4){0.f, 0.f, 0.f, 0.f};
  for (int s = 0; s < count; s += 8) {
    float pm[8], pl[8];
    f32x4 po[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int it = s + u < count ? s + u : count - 1;
      const i64 prow = (i64)(first + it) * CL_Q_HEADS + qh;
      pm[u] = CL_CARG_PM[prow];
      pl[u] = CL_CARG_PL[prow];
      po[u] = *reinterpret_cast<const f32x4*>(CL_CARG_PO + prow * CL_VDIM + d);
    }
    float m_new = m;
#pragma unroll
    for (int u = 0; u < 8; ++u) m_new = fmaxf(m_new, pm[u]);   // (a repeated item's maximum is one the group has anyway)
    const float keep = fast_exp2(m - m_new);
    m = m_new;
    l *= keep;
    o *= keep;
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const float f = s + u < count ? fast_exp2(pm[u] - m) : 0.f;
      l += pl[u] * f;
      o += po[u] * f;
    }
  }
  const float inv = 1.0f / fmaxf(l, 1.0e-30f);
  elem4 r;
#pragma unroll
  for (int i = 0; i < 4; ++i) r[i] = to_elem(o[i] * inv);
  *reinterpret_cast<elem4*>(CL_CARG_OUT + row * CL_VDIM + d) = r;
#if CL_EMIT_LSE
  if (d == 0) CL_CARG_LSE[row] = l > 0.f ? m + fast_log2(l) : CL_NEG_INF;
#endif
}
#elif CL_SPLITS > 1 && CL_EMIT_COMBINE && CL_PO_ELEM
// Combine of partials whose values are stored in the element type (normalised per split, m the
// split's log-sum-exp, l = 1, or 0 with zero values for an empty split): the same rule as below,
// out[row] = sum_s O_s 2^(m_s - m) / sum_s l_s 2^(m_s - m).
// One thread per (row, 8 d): 16-byte loads.
extern "C" __global__ void __launch_bounds__(256)
CL_COMBINE_NAME(CL_COMBINE_PARAMS) {
  const i64 total = (i64)CL_TOTAL_ROWS * (CL_VDIM / 8);
  const i64 idx = (i64)blockIdx.x * 256 + threadIdx.x;
  if (idx >= total) return;
  const i64 row = idx / (CL_VDIM / 8);
  const int d = (int)(idx % (CL_VDIM / 8)) * 8;
  float ms[CL_SPLITS];
  float m = CL_NEG_BIG;
#pragma unroll
  for (int s = 0; s < CL_SPLITS; ++s) {
    ms[s] = CL_CARG_PM[(i64)s * CL_TOTAL_ROWS + row];
    m = fmaxf(m, ms[s]);
  }
  float l = 0.f;
  float o[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) o[i] = 0.f;
#pragma unroll
  for (int s = 0; s < CL_SPLITS; ++s) {
    const i64 prow = (i64)s * CL_TOTAL_ROWS + row;
    const float f = fast_exp2(ms[s] - m);
    l += CL_CARG_PL[prow] * f;
    const elem8 v = as_elem8(ld16(CL_CARG_PO + prow * CL_VDIM + d));
#pragma unroll
    for (int i = 0; i < 8; ++i) o[i] += to_f32(v[i]) * f;
  }
  const float inv = 1.0f / fmaxf(l, 1.0e-30f);
  elem8 r;
#pragma unroll
  for (int i = 0; i < 8; ++i) r[i] = to_elem(o[i] * inv);
  st16(CL_CARG_OUT + row * CL_VDIM + d, as_u32x4(r));
#if CL_EMIT_LSE
  if (d == 0) CL_CARG_LSE[row] = l > 0.f ? m + fast_log2(l) : CL_NEG_INF;
#endif
}
#elif CL_SPLITS > 1 && CL_EMIT_COMBINE
// Combine: out[row] = sum_s O_s 2^(m_s - m) / sum_s l_s 2^(m_s - m).  One thread per (row, 4 d).
extern "C" __global__ void __launch_bounds__(256)
CL_COMBINE_NAME(CL_COMBINE_PARAMS) {
  const i64 total = (i64)CL_TOTAL_ROWS * (CL_VDIM / 4);
  const i64 idx = (i64)blockIdx.x * 256 + threadIdx.x;
  if (idx >= total) return;
  const i64 row = idx / (CL_VDIM / 4);
  const int d = (int)(idx % (CL_VDIM / 4)) * 4;
  float m = CL_NEG_BIG;
#pragma unroll
  for (int s = 0; s < CL_SPLITS; ++s) m = fmaxf(m, CL_CARG_PM[(i64)s * CL_TOTAL_ROWS + row]);
  float l = 0.f;
  f32x4 o = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int s = 0; s < CL_SPLITS; ++s) {
    const i64 prow = (i64)s * CL_TOTAL_ROWS + row;
    const float f = fast_exp2(CL_CARG_PM[prow] - m);
    l += CL_CARG_PL[prow] * f;
    o += *reinterpret_cast<const f32x4*>(CL_CARG_PO + prow * CL_VDIM + d) * f;
  }
  const float inv = 1.0f / fmaxf(l, 1.0e-30f);
  elem4 r;
#pragma unroll
  for (int i = 0; i < 4; ++i) r[i] = to_elem(o[i] * inv);
  *reinterpret_cast<elem4*>(CL_CARG_OUT + row * CL_VDIM + d) = r;
#if CL_EMIT_LSE
  if (d == 0) CL_CARG_LSE[row] = l > 0.f ? m + fast_log2(l) : CL_NEG_INF;
#endif
}
#endif
