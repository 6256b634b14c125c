// ---- split-K combine of the matmul families: C = sum_s P[s] (times the RMSNorm row factor) -----
// One thread per (row, CL_COMBINE_COLS columns).  The kernel is a few MB of traffic at most and
// bound by launch and load latency, so the emitter picks the column count that still gives the
// chip a few hundred workgroups.
//   CL_COMBINE_ROWS   rows of C (batch entries folded in)     CL_N   columns
//   CL_COMBINE_COLS   1, 2 or 4                               CL_NORM / CL_K / CL_EPS  as in the partial
// CL_LORA: C = sum_s P[s] + D * LB with D = sum_s PD[s] (M x CL_R, rounded to the element type as
// the input of the reference's second product is) and LB (CL_R, N).  A workgroup's 256 threads
// share one row of C (the emitter picks the column count so that N / cols is a multiple of
// 256), so the row of D is summed once per workgroup into LDS.
#ifndef CL_LORA
#define CL_LORA 0
#endif
#if CL_SPLITS > 1 && CL_EMIT_COMBINE
extern "C" __global__ void __launch_bounds__(256)
CL_COMBINE_NAME(CL_COMBINE_PARAMS) {
#if CL_LORA
  static_assert((CL_N / CL_COMBINE_COLS) % 256 == 0, "a workgroup of the LoRA combine works on one row");
  __shared__ float mc_d[CL_R];
  {
    const i64 row0 = ((i64)blockIdx.x * 256) / (CL_N / CL_COMBINE_COLS);
    if (threadIdx.x < CL_R) {
      float d = 0.f;
#pragma unroll
      for (int s = 0; s < CL_SPLITS; ++s) d += CL_CARG_PD[((i64)s * CL_COMBINE_ROWS + row0) * CL_R + threadIdx.x];
      mc_d[threadIdx.x] = to_f32(to_elem(d));
    }
    __syncthreads();
  }
#endif
  typedef float mc_f32 __attribute__((ext_vector_type(CL_COMBINE_COLS)));
  typedef elem_t mc_elem __attribute__((ext_vector_type(CL_COMBINE_COLS)));
  const i64 rows = CL_COMBINE_ROWS;
  const i64 total = rows * (CL_N / CL_COMBINE_COLS);
  const i64 idx = (i64)blockIdx.x * 256 + threadIdx.x;
  if (idx >= total) return;
  const i64 row = idx / (CL_N / CL_COMBINE_COLS);
  const int n = (int)(idx % (CL_N / CL_COMBINE_COLS)) * CL_COMBINE_COLS;
  float a[CL_COMBINE_COLS];
#pragma unroll
  for (int r = 0; r < CL_COMBINE_COLS; ++r) a[r] = 0.f;
#if CL_NORM
  float tot = 0.f;
#endif
#pragma unroll
  for (int s = 0; s < CL_SPLITS; ++s) {
    const float* p = CL_CARG_PACC + ((i64)s * rows + row) * CL_N + n;
#if CL_COMBINE_COLS == 1
    a[0] += p[0];
#else
    const mc_f32 v = *reinterpret_cast<const mc_f32*>(p);
#pragma unroll
    for (int r = 0; r < CL_COMBINE_COLS; ++r) a[r] += v[r];
#endif
#if CL_NORM
    tot += CL_CARG_PSS[(i64)s * rows + row];
#endif
  }
#if CL_NORM
  const float rs = fast_rsqrt(tot * (1.0f / CL_K) + CL_EPS);
#else
  const float rs = 1.0f;
#endif
#if CL_LORA
  for (int rr = 0; rr < CL_R; ++rr) {
    const float d = mc_d[rr];
#pragma unroll
    for (int r = 0; r < CL_COMBINE_COLS; ++r) a[r] += d * to_f32(CL_CARG_LB[(i64)rr * CL_N + n + r]);
  }
#endif
#if CL_COMBINE_COLS == 1
  CL_CARG_OUT[row * CL_N + n] = to_elem(a[0] * rs);
#else
  mc_elem y;
#pragma unroll
  for (int r = 0; r < CL_COMBINE_COLS; ++r) y[r] = to_elem(a[r] * rs);
  *reinterpret_cast<mc_elem*>(CL_CARG_OUT + row * CL_N + n) = y;
#endif
}
#endif
