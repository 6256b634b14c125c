// ---- weight-streaming matmul for few rows: Y[M<=64, N] = f(X)[M, K] * W[K, N] ---------------
//
// With M this small the kernel is a pure stream of W out of HBM, so W never touches LDS:
// each wave owns 128 output columns and walks its K range 32 rows at a time.  A lane loads
// an 8(k) x 8(n) block of W as eight 16-byte row segments (sixteen lanes cover 256 contiguous
// bytes of a row), transposes it in registers and feeds eight 16x16x32 MFMAs whose B operands
// are the eight columns of that block; X rows are the A operand, read from L2.
//
// Optional fused RMSNorm (CL_NORM): f(X) = X * gamma (gamma optional), the row sum of squares
// is accumulated from the same X fragments, and the epilogue multiplies row m by
// rsqrt(sumsq[m] / K + eps).  With CL_SPLITS > 1 the block writes f32 partial products (and
// partial sums of squares); the combine kernel adds them up and normalises.
//
//   CL_M, CL_N, CL_K   problem size (K % 32 == 0, N % 8 == 0)
//   CL_WAVES_N         waves side by side along N (each 128 columns)
//   CL_WAVES_K         waves sharing one column slab, splitting the block's K range
//   CL_SPLITS          K splits across workgroups (grid.y)
//   CL_NORM            0 plain, 1 RMSNorm epilogue; CL_GAMMA: 1 when a (K) weight multiplies X
//   CL_EPS             epsilon inside the rsqrt
//   CL_PREFETCH        steps of loads in flight ahead of the one being computed (1..3)
//
// CL_LORA: Y = X * W + (X * LA) * LB with LA (K, CL_R) and LB (CL_R, N).  The rank-R
// product D = X * LA rides along: the lanes of the first CL_R / 8 column groups load their 8x8
// blocks of LA with the W blocks (same ring, same transpose, eight more MFMAs per step into a
// second accumulator set of which only those column groups mean anything), D is reduced over the
// K-sharing waves with the main accumulators, rounded to the element type like the input of the
// reference's second product, parked in LDS, and the epilogue adds D * LB to each lane's outputs
// with plain multiply-adds (CL_R per output).  Split over K (CL_SPLITS > 1) the rank update cannot
// happen here (it needs all of D): the first column slab's workgroups write their partial sums
// of D beside the partial products (CL_ARG_PD[split][M][CL_R]) and the combine applies it.

#define SK_MT ((CL_M + 15) / 16)
#define SK_COLS 128
#define SK_STEP 32
#define SK_THREADS (CL_WAVES_N * CL_WAVES_K * 64)

#ifndef CL_PREFETCH
#define CL_PREFETCH 2
#endif
#ifndef CL_LORA
#define CL_LORA 0
#endif
#if CL_LORA
static_assert(CL_R % 8 == 0 && CL_R <= 128 && !CL_NORM, "LoRA: rank in whole 8-column blocks");
#endif
// Everything one 32-row step needs, as loaded: the lane's 8x8 block of W, its X fragments
// (lane (c, g) holds X[16 mt + c][k0 + 8 g .. +8]) and the matching gamma chunk.  X and gamma
// travel with the W block on purpose: a small load issued on its own in the loop would sit
// behind the W prefetches in the in-order load queue and make every step wait for them.
struct SkTile {
  u32x4 w[8];
  u32x4 x[SK_MT];
#if CL_NORM && CL_GAMMA
  u32x4 gm;
#endif
#if CL_LORA
  u32x4 la[8];
#endif
};

CL_DEVICE void sk_load(const elem_t* __restrict__ W, const elem_t* __restrict__ X, const elem_t* __restrict__ G,
                       const elem_t* __restrict__ LA, int k0, int ncol, int c, int g, SkTile& t) {
#pragma unroll
  for (int e = 0; e < 8; ++e) t.w[e] = ld16(W + (i64)(k0 + 8 * g + e) * CL_N + ncol);
#pragma unroll
  for (int mt = 0; mt < SK_MT; ++mt) {
    const int m = 16 * mt + c;
    t.x[mt] = ld16(X + (i64)(m < CL_M ? m : CL_M - 1) * CL_K + k0 + 8 * g);   // rows past M: masked when used
  }
#if CL_NORM && CL_GAMMA
  t.gm = ld16(G + k0 + 8 * g);
#else
  (void)G;
#endif
#if CL_LORA
#pragma unroll
  for (int e = 0; e < 8; ++e)   // (only the lanes of the first CL_R / 8 column groups fetch anything)
    t.la[e] = 8 * c < CL_R ? ld16(LA + (i64)(k0 + 8 * g + e) * CL_R + 8 * c) : (u32x4){0u, 0u, 0u, 0u};
#else
  (void)LA;
#endif
}

#if CL_EMIT_PARTIAL
extern "C" __global__ void __launch_bounds__(SK_THREADS)
CL_PARTIAL_NAME(CL_PARTIAL_PARAMS) {
  // (readfirstlane: everything derived from the wave index is uniform and stays in scalar registers)
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int c = lane & 15, g = lane >> 4;
  const int wn = wave % CL_WAVES_N, wk = wave / CL_WAVES_N;
  const int split = blockIdx.y;

  // columns of this wave; the last slab may hang over N: loads are clamped, stores masked
  const int n_base = (blockIdx.x * CL_WAVES_N + wn) * SK_COLS;
  int ncol = n_base + 8 * c;
  const bool col_live = ncol < CL_N;
  ncol = col_live ? ncol : CL_N - 8;

  // K range: split -> waves_k, contiguous chunks of whole 32-row steps
  constexpr int steps_total = CL_K / SK_STEP;
  constexpr int steps_per_split = (steps_total + CL_SPLITS - 1) / CL_SPLITS;
  constexpr int steps_per_wave = (steps_per_split + CL_WAVES_K - 1) / CL_WAVES_K;
  int s_begin = split * steps_per_split + wk * steps_per_wave;
  int s_end = s_begin + steps_per_wave;
  {
    int lim = (split + 1) * steps_per_split;
    lim = lim < steps_total ? lim : steps_total;
    s_end = s_end < lim ? s_end : lim;
  }

  f32x4 acc[SK_MT][8];
#pragma unroll
  for (int mt = 0; mt < SK_MT; ++mt)
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[mt][j] = (f32x4){0.f, 0.f, 0.f, 0.f};
  float ss[SK_MT];
#pragma unroll
  for (int mt = 0; mt < SK_MT; ++mt) ss[mt] = 0.f;
#if CL_LORA
  f32x4 dacc[SK_MT][8];        // dacc[mt][j][r] = D[16 mt + 4 g + r][8 c + j] in the lanes with 8 c < CL_R
#pragma unroll
  for (int mt = 0; mt < SK_MT; ++mt)
#pragma unroll
    for (int j = 0; j < 8; ++j) dacc[mt][j] = (f32x4){0.f, 0.f, 0.f, 0.f};
#endif

  // Ring of CL_PREFETCH + 1 register tiles: while step n is in the matrix cores the loads of
  // steps n+1 .. n+CL_PREFETCH are in flight.
#if CL_NORM && CL_GAMMA
  const elem_t* gamma_ptr = CL_ARG_GAMMA;
#else
  const elem_t* gamma_ptr = nullptr;
#endif
#if CL_LORA
  const elem_t* la_ptr = CL_ARG_LA;
#else
  const elem_t* la_ptr = nullptr;
#endif
  SkTile ring[CL_PREFETCH + 1];
  // one step on the tile `cur`: row sums of squares, gamma, 8x8 transpose of W, eight MFMAs per row tile
#define SK_CONSUME(cur)                                                                   \
  {                                                                                       \
    elem8 xa[SK_MT];                                                                      \
    _Pragma("unroll") for (int mt = 0; mt < SK_MT; ++mt) {                                \
      u32x4 raw = (cur).x[mt];                                                            \
      if (16 * mt + c >= CL_M) raw = (u32x4){0u, 0u, 0u, 0u};                             \
      elem8 x = as_elem8(raw);                                                            \
      SK_NORM_X(x, mt, cur)                                                               \
      xa[mt] = x;                                                                         \
    }                                                                                     \
    u32x4 wt[8];                                                                          \
    transpose8x8((cur).w, wt);                                                            \
    _Pragma("unroll") for (int j = 0; j < 8; ++j)                                         \
      _Pragma("unroll") for (int mt = 0; mt < SK_MT; ++mt)                                \
        acc[mt][j] = mfma16(xa[mt], as_elem8(wt[j]), acc[mt][j]);                         \
    SK_LORA_STEP(cur)                                                                     \
  }
#if CL_LORA
#define SK_LORA_STEP(cur)                                                                 \
    {                                                                                     \
      u32x4 lt[8];                                                                        \
      transpose8x8((cur).la, lt);                                                         \
      _Pragma("unroll") for (int j = 0; j < 8; ++j)                                       \
        _Pragma("unroll") for (int mt = 0; mt < SK_MT; ++mt)                              \
          dacc[mt][j] = mfma16(xa[mt], as_elem8(lt[j]), dacc[mt][j]);                     \
    }
#else
#define SK_LORA_STEP(cur)
#endif
#if CL_NORM
#if CL_GAMMA
#define SK_GAMMA_X(x, cur)                                                                \
  {                                                                                       \
    const elem8 gm = as_elem8((cur).gm);                                                  \
    _Pragma("unroll") for (int i = 0; i < 8; ++i) x[i] = to_elem(to_f32(x[i]) * to_f32(gm[i])); \
  }
#else
#define SK_GAMMA_X(x, cur)
#endif
#define SK_NORM_X(x, mt, cur)                                                             \
  _Pragma("unroll") for (int i = 0; i < 8; ++i) {                                         \
    const float xf = to_f32(x[i]);                                                        \
    ss[mt] += xf * xf;                                                                    \
  }                                                                                       \
  SK_GAMMA_X(x, cur)
#else
#define SK_NORM_X(x, mt, cur)
#endif

  if constexpr (steps_total % (CL_SPLITS * CL_WAVES_K) == 0 && steps_per_wave <= 32) {
    // every wave has exactly steps_per_wave steps: the whole walk is straight-line code, each
    // load issued CL_PREFETCH steps ahead of its use and none past the end
#pragma unroll
    for (int i = 0; i < CL_PREFETCH && i < steps_per_wave; ++i)
      sk_load(CL_ARG_W, CL_ARG_X, gamma_ptr, la_ptr, (s_begin + i) * SK_STEP, ncol, c, g, ring[i % (CL_PREFETCH + 1)]);
#pragma unroll
    for (int i = 0; i < steps_per_wave; ++i) {
      if (i + CL_PREFETCH < steps_per_wave)
        sk_load(CL_ARG_W, CL_ARG_X, gamma_ptr, la_ptr, (s_begin + i + CL_PREFETCH) * SK_STEP, ncol, c, g,
                ring[(i + CL_PREFETCH) % (CL_PREFETCH + 1)]);
      SK_CONSUME(ring[i % (CL_PREFETCH + 1)])
    }
  } else {
    // Ragged ranges: prefetch loads are issued unconditionally, a step past the end clamped onto
    // the wave's last step (an L2 hit, never consumed), so the load counter is the same on every
    // path and the waits stay exact.
    const int last_step = s_end - 1;
    if (s_begin < s_end) {
#pragma unroll
      for (int i = 0; i < CL_PREFETCH; ++i) {
        int sidx = s_begin + i;
        sidx = sidx < last_step ? sidx : last_step;
        sk_load(CL_ARG_W, CL_ARG_X, gamma_ptr, la_ptr, sidx * SK_STEP, ncol, c, g, ring[i]);
      }
    }
    for (int base = s_begin; base < s_end; base += CL_PREFETCH + 1) {
#pragma unroll
      for (int r = 0; r <= CL_PREFETCH; ++r) {
        const int s = base + r;
        if (s >= s_end) break;
        int ahead = s + CL_PREFETCH;
        ahead = ahead < last_step ? ahead : last_step;
        sk_load(CL_ARG_W, CL_ARG_X, gamma_ptr, la_ptr, ahead * SK_STEP, ncol, c, g, ring[(r + CL_PREFETCH) % (CL_PREFETCH + 1)]);
        SK_CONSUME(ring[r])
      }
    }
  }

  // ---- reduce across the waves that share a column slab ------------------------------------
  // acc[mt][j][r] = Y[16 mt + 4 g + r][n_base + 8 c + j]
#if CL_NORM
#pragma unroll
  for (int mt = 0; mt < SK_MT; ++mt) {
    ss[mt] += lane_xor(ss[mt], lane, 16);
    ss[mt] += lane_xor(ss[mt], lane, 32);
  }
#endif
  extern __shared__ float sk_lds[];
  float* sh_acc = sk_lds;                                     // [WAVES_K-1][WAVES_N][MT*8*4][64]
  float* sh_ss = sk_lds + (CL_WAVES_K - 1) * CL_WAVES_N * SK_MT * 32 * 64;  // [WAVES_K][MT*16]
#if CL_LORA
  float* sh_dacc = sh_ss + CL_WAVES_K * SK_MT * 16 + 4;       // like sh_acc, for the rank-R accumulators
  float* sh_d = sh_dacc + (CL_WAVES_K - 1) * CL_WAVES_N * SK_MT * 32 * 64;  // [WAVES_N][16 MT][CL_R]
#endif
#if CL_WAVES_K > 1
  if (wk > 0) {
    float* dst = sh_acc + ((i64)((wk - 1) * CL_WAVES_N + wn) * SK_MT * 32) * 64;
#pragma unroll
    for (int mt = 0; mt < SK_MT; ++mt)
#pragma unroll
      for (int j = 0; j < 8; ++j)
#pragma unroll
        for (int r = 0; r < 4; ++r) dst[((mt * 8 + j) * 4 + r) * 64 + lane] = acc[mt][j][r];
#if CL_LORA
    float* ddst = sh_dacc + ((i64)((wk - 1) * CL_WAVES_N + wn) * SK_MT * 32) * 64;
#pragma unroll
    for (int mt = 0; mt < SK_MT; ++mt)
#pragma unroll
      for (int j = 0; j < 8; ++j)
#pragma unroll
        for (int r = 0; r < 4; ++r) ddst[((mt * 8 + j) * 4 + r) * 64 + lane] = dacc[mt][j][r];
#endif
  }
#endif
#if CL_NORM
  if (wn == 0 && g == 0) {
#pragma unroll
    for (int mt = 0; mt < SK_MT; ++mt) sh_ss[wk * SK_MT * 16 + mt * 16 + c] = ss[mt];
  }
#endif
  __syncthreads();
#if !CL_LORA
  if (wk != 0) {
    return;
  }
#endif
#if CL_WAVES_K > 1
  if (wk == 0) {
#pragma unroll
    for (int w = 1; w < CL_WAVES_K; ++w) {
      const float* src = sh_acc + ((i64)((w - 1) * CL_WAVES_N + wn) * SK_MT * 32) * 64;
#pragma unroll
      for (int mt = 0; mt < SK_MT; ++mt)
#pragma unroll
        for (int j = 0; j < 8; ++j)
#pragma unroll
          for (int r = 0; r < 4; ++r) acc[mt][j][r] += src[((mt * 8 + j) * 4 + r) * 64 + lane];
#if CL_LORA
      const float* dsrc = sh_dacc + ((i64)((w - 1) * CL_WAVES_N + wn) * SK_MT * 32) * 64;
#pragma unroll
      for (int mt = 0; mt < SK_MT; ++mt)
#pragma unroll
        for (int j = 0; j < 8; ++j)
#pragma unroll
          for (int r = 0; r < 4; ++r) dacc[mt][j][r] += dsrc[((mt * 8 + j) * 4 + r) * 64 + lane];
#endif
    }
  }
#endif
#if CL_LORA && CL_SPLITS > 1
  if (wk != 0) return;
  if (blockIdx.x == 0 && wn == 0 && 8 * c < CL_R) {
#pragma unroll
    for (int mt = 0; mt < SK_MT; ++mt)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int m = 16 * mt + 4 * g + r;
        if (m >= CL_M) continue;
        float* drow = CL_ARG_PD + ((i64)split * CL_M + m) * CL_R + 8 * c;
        *reinterpret_cast<f32x4*>(drow) = (f32x4){dacc[mt][0][r], dacc[mt][1][r], dacc[mt][2][r], dacc[mt][3][r]};
        *reinterpret_cast<f32x4*>(drow + 4) = (f32x4){dacc[mt][4][r], dacc[mt][5][r], dacc[mt][6][r], dacc[mt][7][r]};
      }
  }
#elif CL_LORA
  // D (rounded to the element type, as the input of a second product is) goes to LDS for this
  // wave's epilogue; the workgroup-wide barrier is the simplest fence between its lanes
  if (wk == 0 && 8 * c < CL_R) {
#pragma unroll
    for (int mt = 0; mt < SK_MT; ++mt)
#pragma unroll
      for (int j = 0; j < 8; ++j)
#pragma unroll
        for (int r = 0; r < 4; ++r)
          sh_d[((wn * SK_MT + mt) * 16 + 4 * g + r) * CL_R + 8 * c + j] = to_f32(to_elem(dacc[mt][j][r]));
  }
  __syncthreads();
  if (wk != 0) return;
  for (int rr = 0; rr < CL_R; ++rr) {
    const elem8 bv = as_elem8(ld16(CL_ARG_LB + (i64)rr * CL_N + ncol));
#pragma unroll
    for (int mt = 0; mt < SK_MT; ++mt)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float d = sh_d[((wn * SK_MT + mt) * 16 + 4 * g + r) * CL_R + rr];
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[mt][j][r] += d * to_f32(bv[j]);
      }
  }
#endif

  // ---- epilogue ----------------------------------------------------------------------------
#pragma unroll
  for (int mt = 0; mt < SK_MT; ++mt) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int m = 16 * mt + 4 * g + r;
      if (m >= CL_M) continue;
#if CL_NORM
      float tot = 0.f;
#pragma unroll
      for (int w = 0; w < CL_WAVES_K; ++w) tot += sh_ss[w * SK_MT * 16 + mt * 16 + 4 * g + r];
#endif
#if CL_SPLITS > 1
      float* prow = CL_ARG_PACC + ((i64)split * CL_M + m) * CL_N + n_base + 8 * c;
      if (col_live) {
        *reinterpret_cast<f32x4*>(prow) = (f32x4){acc[mt][0][r], acc[mt][1][r], acc[mt][2][r], acc[mt][3][r]};
        *reinterpret_cast<f32x4*>(prow + 4) = (f32x4){acc[mt][4][r], acc[mt][5][r], acc[mt][6][r], acc[mt][7][r]};
      }
#if CL_NORM
      if (blockIdx.x == 0 && wn == 0 && c == 0) CL_ARG_PSS[(i64)split * CL_M + m] = tot;
#endif
#else
#if CL_NORM
      const float rs = fast_rsqrt(tot * (1.0f / CL_K) + CL_EPS);
#else
      const float rs = 1.0f;
#endif
      elem8 y;
#pragma unroll
      for (int j = 0; j < 8; ++j) y[j] = to_elem(acc[mt][j][r] * rs);
      if (col_live) st16(CL_ARG_OUT + (i64)m * CL_N + n_base + 8 * c, as_u32x4(y));
#endif
    }
  }
}
#endif  // CL_EMIT_PARTIAL
