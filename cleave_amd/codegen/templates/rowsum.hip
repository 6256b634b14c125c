// ---- row reductions over the last axis: out[m] = sum_n x[m][n], or out[m][n] = x[m][n] / sum_n x[m][n]
//
// One wave per row, CL_ROWS_PER_BLOCK rows per workgroup: a lane reads 16 bytes (8 elements) of
// every 1 KiB of the row, adds them up in fp32, the wave folds the 64 partial sums with cross-lane
// reads.  CL_DIV: each element divided by the sum; a row of up to 8192 elements in whole 512-element
// pieces stays in the lane's registers between the two passes (all of its loads in flight at once,
// nothing read twice), a longer or ragged one is read a second time (it is still in L2).  Pure HBM
// streaming: nothing here is worth the matrix unit.
//
//   CL_M rows, CL_N columns (multiple of 8), CL_ROWS_PER_BLOCK (1, 2 or 4), CL_DIV

#if CL_EMIT_PARTIAL
extern "C" __global__ void __launch_bounds__(64 * CL_ROWS_PER_BLOCK)
CL_PARTIAL_NAME(CL_PARTIAL_PARAMS) {
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const i64 row = (i64)blockIdx.x * CL_ROWS_PER_BLOCK + wave;
  if (row >= CL_M) return;
  const elem_t* src = CL_ARG_X + row * CL_N;
  float sum = 0.f;
#if CL_DIV && CL_N % 512 == 0 && CL_N <= 8192
  {
    constexpr int PIECES = CL_N / 512;
    u32x4 raw[PIECES];
#pragma unroll
    for (int u = 0; u < PIECES; ++u) raw[u] = ld16(src + 8 * lane + 512 * u);
#pragma unroll
    for (int u = 0; u < PIECES; ++u) {
      const elem8 v = as_elem8(raw[u]);
#pragma unroll
      for (int i = 0; i < 8; ++i) sum += to_f32(v[i]);
    }
#pragma unroll
    for (int mask = 1; mask < 64; mask <<= 1) sum += lane_xor(sum, lane, mask);
    const float inv = 1.0f / sum;
    elem_t* dst = CL_ARG_OUT + row * CL_N;
#pragma unroll
    for (int u = 0; u < PIECES; ++u) {
      elem8 v = as_elem8(raw[u]);
#pragma unroll
      for (int i = 0; i < 8; ++i) v[i] = to_elem(to_f32(v[i]) * inv);
      st16(dst + 8 * lane + 512 * u, as_u32x4(v));
    }
    return;
  }
#endif
  // four independent loads per trip keep the memory pipe fed; chunks past the row's end read its last chunk with weight 0
  for (int n0 = 8 * lane; n0 < CL_N; n0 += 4 * 512) {
    u32x4 raw[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int n = n0 + 512 * u;
      raw[u] = ld16(src + (n < CL_N ? n : CL_N - 8));
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      if (n0 + 512 * u >= CL_N) continue;
      const elem8 v = as_elem8(raw[u]);
#pragma unroll
      for (int i = 0; i < 8; ++i) sum += to_f32(v[i]);
    }
  }
#pragma unroll
  for (int mask = 1; mask < 64; mask <<= 1) sum += lane_xor(sum, lane, mask);
#if CL_DIV
  const float inv = 1.0f / sum;
  elem_t* dst = CL_ARG_OUT + row * CL_N;
  for (int n0 = 8 * lane; n0 < CL_N; n0 += 512) {
    elem8 v = as_elem8(ld16(src + n0));
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = to_elem(to_f32(v[i]) * inv);
    st16(dst + n0, as_u32x4(v));
  }
#else
  if (lane == 0) CL_ARG_OUT[row] = to_elem(sum);
#endif
}
#endif  // CL_EMIT_PARTIAL
