// ---- rows of a (rows, width) tensor scaled by rsqrt(mean(x^2) + eps), written in the element type ----
// The keys of a QK-norm attention normalised once, ahead of the attention kernel, instead of by
// every workgroup that reads them (an attention kernel over S queries reads every key S / 128
// times).  One lane per 16-byte chunk of a row; the lanes of a row (width / 8, a power of two of
// at most 32) add up their squares through lane exchanges.
//   CL_KPRE_ROWS  rows     CL_HEAD_DIM  width     CL_KNORM_EPS  epsilon inside the root
//   CL_KPRE_SRC / CL_KPRE_DST  the tensor and its normalised copy
#if CL_EMIT_KPRE
extern "C" __global__ void __launch_bounds__(256)
CL_KPRE_NAME(CL_KPRE_PARAMS) {
  constexpr int LANES = CL_HEAD_DIM / 8;
  static_assert(LANES >= 1 && LANES <= 32 && (LANES & (LANES - 1)) == 0, "a row's chunks are a power of two of lanes within a wave");
  const int lane = threadIdx.x & 63;
  const i64 idx = (i64)blockIdx.x * 256 + threadIdx.x;
  const i64 rows = CL_KPRE_ROWS;
  const i64 row = idx / LANES;
  const int chunk = (int)(idx % LANES);
  const i64 r = row < rows ? row : rows - 1;            // (whole waves take part in the lane exchanges)
  const elem8 x = as_elem8(ld16(CL_KPRE_SRC + r * CL_HEAD_DIM + 8 * chunk));
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i) ss += to_f32(x[i]) * to_f32(x[i]);
#pragma unroll
  for (int d = 1; d < LANES; d <<= 1) ss += lane_xor(ss, lane, d);
  const float f = fast_rsqrt(ss * (1.0f / CL_HEAD_DIM) + CL_KNORM_EPS);
  elem8 y;
#pragma unroll
  for (int i = 0; i < 8; ++i) y[i] = to_elem(to_f32(x[i]) * f);
  if (row < rows) st16(CL_KPRE_DST + row * CL_HEAD_DIM + 8 * chunk, as_u32x4(y));
}
#endif
