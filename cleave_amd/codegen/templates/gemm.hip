// ---- LDS-tiled MFMA matmul: C[M, N] = f(A)[M, K] * B[K, N], f16 / bf16 in, f32 accumulate ----
//
// A workgroup owns a BM x BN tile of C and walks K in steps of BK.  Both operands are kept in
// LDS with the contraction axis minor (padded rows), so a matrix-core operand is one 16-byte
// LDS read.  An operand whose global layout already has K minor is copied chunk by chunk; one
// whose K is the major axis (B given as (K, N), A given as (K, M)) is loaded as 8x8 blocks and
// transposed in registers on its way into LDS.  Global loads of step i+1 are in flight while
// the matrix cores work on step i (two LDS stages, one barrier per step).
//
//   CL_M CL_N CL_K            problem size per batch entry (K % (CL_SPLITS*CL_BK) == 0)
//   CL_BM CL_BN CL_BK         workgroup tile;  CL_WM x CL_WN waves, each (BM/WM) x (BN/WN)
//   CL_TRANS_A / CL_TRANS_B   1 when the operand is stored with K as its major / minor axis
//                             opposite to the default (A: (M,K), B: (K,N))
//   CL_BATCH_A CL_BATCH_B     batch counts (grouped broadcast: the larger is the grid's)
//   CL_SPLITS                 split-K factor: partial f32 tiles go to CL_ARG_PACC[split]
//   CL_NORM / CL_GAMMA / CL_EPS   fused RMSNorm of A's rows (see the skinny kernel)

#define GM_THREADS (CL_WM * CL_WN * 64)
#define GM_TM (CL_BM / CL_WM / 16)
#define GM_TN (CL_BN / CL_WN / 16)
#define GM_LD (CL_BK + 8)                       // LDS row pitch in elements (16-byte pad)
#define GM_KC (CL_BK / 8)                       // 16-byte chunks along K per tile row
#define GM_BATCH (CL_BATCH_A > CL_BATCH_B ? CL_BATCH_A : CL_BATCH_B)

// ---- K-minor operand: rows x BK tile, chunk q -> (row q / KC, chunk q % KC) -------------------
template <int ROWS>
struct GmDirect {
  static constexpr int PER = (ROWS * GM_KC + GM_THREADS - 1) / GM_THREADS;
  u32x4 v[PER];
  CL_METHOD void load(const elem_t* __restrict__ base, i64 pitch, int row0, int row_lim, int k0) {
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int q = threadIdx.x + i * GM_THREADS;
      int row = row0 + q / GM_KC;
      row = row < row_lim ? row : row_lim - 1;
      if (ROWS * GM_KC % GM_THREADS == 0 || q < ROWS * GM_KC)
        v[i] = ld16(base + (i64)row * pitch + k0 + 8 * (q % GM_KC));
    }
  }
  CL_METHOD void store(elem_t* lds) const {
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int q = threadIdx.x + i * GM_THREADS;
      if (ROWS * GM_KC % GM_THREADS == 0 || q < ROWS * GM_KC)
        *reinterpret_cast<u32x4*>(lds + (q / GM_KC) * GM_LD + 8 * (q % GM_KC)) = v[i];
    }
  }
};

// ---- K-major operand: BK x COLS tile as 8x8 blocks, block q -> (k-block q / NB, col-block q % NB)
template <int COLS>
struct GmTransposed {
  static constexpr int NB = COLS / 8;
  static constexpr int BLOCKS = GM_KC * NB;
  static constexpr int PER = (BLOCKS + GM_THREADS - 1) / GM_THREADS;
  u32x4 v[PER][8];
  CL_METHOD void load(const elem_t* __restrict__ base, i64 pitch, int col0, int col_lim, int k0) {
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int q = threadIdx.x + i * GM_THREADS;
      if (BLOCKS % GM_THREADS == 0 || q < BLOCKS) {
        int col = col0 + 8 * (q % NB);
        col = col < col_lim - 8 ? col : col_lim - 8;
        const elem_t* p = base + (i64)(k0 + 8 * (q / NB)) * pitch + col;
#pragma unroll
        for (int e = 0; e < 8; ++e) v[i][e] = ld16(p + (i64)e * pitch);
      }
    }
  }
  CL_METHOD void store(elem_t* lds) const {
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int q = threadIdx.x + i * GM_THREADS;
      if (BLOCKS % GM_THREADS == 0 || q < BLOCKS) {
        u32x4 t[8];
        transpose8x8(v[i], t);
        elem_t* dst = lds + (8 * (q % NB)) * GM_LD + 8 * (q / NB);
#pragma unroll
        for (int j = 0; j < 8; ++j) *reinterpret_cast<u32x4*>(dst + j * GM_LD) = t[j];
      }
    }
  }
};

#if CL_EMIT_PARTIAL
extern "C" __global__ void __launch_bounds__(GM_THREADS)
CL_PARTIAL_NAME(CL_PARTIAL_PARAMS) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int c = lane & 15, g = lane >> 4;
  const int wm = wave / CL_WN, wn = wave % CL_WN;
  const int m0 = blockIdx.y * CL_BM, n0 = blockIdx.x * CL_BN;
  const int batch = blockIdx.z / CL_SPLITS, split = blockIdx.z % CL_SPLITS;
  constexpr int k_per_split = CL_K / CL_SPLITS;
  const int k_begin = split * k_per_split;
  constexpr int KT = k_per_split / CL_BK;

  const elem_t* A = CL_ARG_A + (i64)(batch / (GM_BATCH / CL_BATCH_A)) * CL_M * CL_K;
  const elem_t* B = CL_ARG_B + (i64)(batch / (GM_BATCH / CL_BATCH_B)) * CL_K * CL_N;

  extern __shared__ __attribute__((aligned(16))) unsigned char gm_lds_raw[];
  elem_t* lds = reinterpret_cast<elem_t*>(gm_lds_raw);
  constexpr int A_STAGE = CL_BM * GM_LD, B_STAGE = CL_BN * GM_LD;
  elem_t* As = lds;                      // [2][BM][LD]
  elem_t* Bs = lds + 2 * A_STAGE;        // [2][BN][LD]
#if CL_NORM
  float* row_ss = reinterpret_cast<float*>(lds + 2 * A_STAGE + 2 * B_STAGE);  // [BM]
  for (int i = threadIdx.x; i < CL_BM; i += GM_THREADS) row_ss[i] = 0.f;
#endif

#if CL_TRANS_A
  GmTransposed<CL_BM> la;
#define GM_LOAD_A(kk) la.load(A, CL_M, m0, CL_M, (kk))
#else
  GmDirect<CL_BM> la;
#define GM_LOAD_A(kk) la.load(A, CL_K, m0, CL_M, (kk))
#endif
#if CL_TRANS_B
  GmDirect<CL_BN> lb;
#define GM_LOAD_B(kk) lb.load(B, CL_K, n0, CL_N, (kk))
#else
  GmTransposed<CL_BN> lb;
#define GM_LOAD_B(kk) lb.load(B, CL_N, n0, CL_N, (kk))
#endif

  f32x4 acc[GM_TM][GM_TN];
#pragma unroll
  for (int i = 0; i < GM_TM; ++i)
#pragma unroll
    for (int j = 0; j < GM_TN; ++j) acc[i][j] = (f32x4){0.f, 0.f, 0.f, 0.f};

#if CL_NORM && !CL_TRANS_A
  float ss_local[GmDirect<CL_BM>::PER];
#pragma unroll
  for (int i = 0; i < GmDirect<CL_BM>::PER; ++i) ss_local[i] = 0.f;
  // sum of squares of the raw rows, then gamma folded into the tile on its way to LDS
#define GM_NORM_A(kk)                                                               \
  _Pragma("unroll") for (int i = 0; i < GmDirect<CL_BM>::PER; ++i) {               \
    elem8 x = as_elem8(la.v[i]);                                                    \
    _Pragma("unroll") for (int e = 0; e < 8; ++e) {                                \
      const float xf = to_f32(x[e]);                                                \
      ss_local[i] += xf * xf;                                                       \
    }                                                                               \
    GM_GAMMA_A(kk)                                                                  \
    la.v[i] = as_u32x4(x);                                                          \
  }
#if CL_GAMMA
#define GM_GAMMA_A(kk)                                                                              \
  {                                                                                                 \
    const int q = threadIdx.x + i * GM_THREADS;                                                     \
    elem8 gm = as_elem8(ld16(CL_ARG_GAMMA + (kk) + 8 * (q % GM_KC)));                               \
    _Pragma("unroll") for (int e = 0; e < 8; ++e) x[e] = to_elem(to_f32(x[e]) * to_f32(gm[e]));    \
  }
#else
#define GM_GAMMA_A(kk)
#endif
#else
#define GM_NORM_A(kk)
#endif

  GM_LOAD_A(k_begin);
  GM_LOAD_B(k_begin);
  GM_NORM_A(k_begin)
  la.store(As);
  lb.store(Bs);
  __syncthreads();

  for (int kt = 0; kt < KT; ++kt) {
    const int cur = kt & 1;
    if (kt + 1 < KT) {
      GM_LOAD_A(k_begin + (kt + 1) * CL_BK);
      GM_LOAD_B(k_begin + (kt + 1) * CL_BK);
    }
    const elem_t* a_tile = As + cur * A_STAGE + (wm * (CL_BM / CL_WM) + c) * GM_LD + 8 * g;
    const elem_t* b_tile = Bs + cur * B_STAGE + (wn * (CL_BN / CL_WN) + c) * GM_LD + 8 * g;
#pragma unroll
    for (int kk = 0; kk < CL_BK; kk += 32) {
      elem8 af[GM_TM], bf[GM_TN];
#pragma unroll
      for (int i = 0; i < GM_TM; ++i) af[i] = *reinterpret_cast<const elem8*>(a_tile + 16 * i * GM_LD + kk);
#pragma unroll
      for (int j = 0; j < GM_TN; ++j) bf[j] = *reinterpret_cast<const elem8*>(b_tile + 16 * j * GM_LD + kk);
      // rows of the MFMA result follow its first operand: feeding B first leaves each lane
      // with four consecutive columns of one row of C
#pragma unroll
      for (int i = 0; i < GM_TM; ++i)
#pragma unroll
        for (int j = 0; j < GM_TN; ++j) acc[i][j] = mfma16(bf[j], af[i], acc[i][j]);
    }
    if (kt + 1 < KT) {
      GM_NORM_A(k_begin + (kt + 1) * CL_BK)
      la.store(As + (cur ^ 1) * A_STAGE);
      lb.store(Bs + (cur ^ 1) * B_STAGE);
    }
    __syncthreads();
  }

#if CL_NORM && !CL_TRANS_A
#pragma unroll
  for (int i = 0; i < GmDirect<CL_BM>::PER; ++i) {
    const int q = threadIdx.x + i * GM_THREADS;
    if (CL_BM * GM_KC % GM_THREADS == 0 || q < CL_BM * GM_KC) atomicAdd(&row_ss[q / GM_KC], ss_local[i]);
  }
  __syncthreads();
#endif

  // ---- epilogue: acc[i][j][r] = C[m0 + wm*.. + 16 i + c][n0 + wn*.. + 16 j + 4 g + r] --------
#pragma unroll
  for (int i = 0; i < GM_TM; ++i) {
    const int ml = wm * (CL_BM / CL_WM) + 16 * i + c;
    const int m = m0 + ml;
    if (m >= CL_M) continue;
#if CL_NORM
    const float tot = row_ss[ml];
#endif
#pragma unroll
    for (int j = 0; j < GM_TN; ++j) {
      const int n = n0 + wn * (CL_BN / CL_WN) + 16 * j + 4 * g;
      if (n >= CL_N) continue;
#if CL_SPLITS > 1
      *reinterpret_cast<f32x4*>(CL_ARG_PACC + (((i64)split * GM_BATCH + batch) * CL_M + m) * CL_N + n) = acc[i][j];
#if CL_NORM
      if (blockIdx.x == 0 && wn == 0 && j == 0 && g == 0) CL_ARG_PSS[((i64)split * GM_BATCH + batch) * CL_M + m] = tot;
#endif
#else
#if CL_NORM
      const float rs = fast_rsqrt(tot * (1.0f / CL_K) + CL_EPS);
#else
      const float rs = 1.0f;
#endif
      elem4 y;
#pragma unroll
      for (int r = 0; r < 4; ++r) y[r] = to_elem(acc[i][j][r] * rs);
      *reinterpret_cast<elem4*>(CL_ARG_OUT + ((i64)batch * CL_M + m) * CL_N + n) = y;
#endif
    }
  }
}
#endif  // CL_EMIT_PARTIAL

#if CL_SPLITS > 1 && CL_EMIT_COMBINE
// Combine: C = sum_s P[s] (times the RMSNorm row factor).  Four columns per thread.
extern "C" __global__ void __launch_bounds__(256)
CL_COMBINE_NAME(CL_COMBINE_PARAMS) {
  const i64 rows = (i64)GM_BATCH * CL_M;
  const i64 total = rows * (CL_N / 4);
  const i64 idx = (i64)blockIdx.x * 256 + threadIdx.x;
  if (idx >= total) return;
  const i64 row = idx / (CL_N / 4);
  const int n = (int)(idx % (CL_N / 4)) * 4;
  f32x4 a = (f32x4){0.f, 0.f, 0.f, 0.f};
#if CL_NORM
  float tot = 0.f;
#endif
#pragma unroll
  for (int s = 0; s < CL_SPLITS; ++s) {
    a += *reinterpret_cast<const f32x4*>(CL_CARG_PACC + ((i64)s * rows + row) * CL_N + n);
#if CL_NORM
    tot += CL_CARG_PSS[(i64)s * rows + row];
#endif
  }
#if CL_NORM
  const float rs = fast_rsqrt(tot * (1.0f / CL_K) + CL_EPS);
#else
  const float rs = 1.0f;
#endif
  elem4 y;
#pragma unroll
  for (int r = 0; r < 4; ++r) y[r] = to_elem(a[r] * rs);
  *reinterpret_cast<elem4*>(CL_CARG_OUT + row * CL_N + n) = y;
}
#endif
