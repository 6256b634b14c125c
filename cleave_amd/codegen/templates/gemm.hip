// ---- LDS-tiled MFMA matmul: C[M, N] = f(A)[M, K] * B[K, N], f16 / bf16 in, f32 accumulate ----
//
// A workgroup owns a BM x BN tile of C and walks K in steps of BK.  Both operands are kept in
// LDS with the contraction axis minor (padded rows), so a matrix-core operand is one 16-byte
// LDS read.  An operand whose global layout already has K minor is copied chunk by chunk; one
// whose K is the major axis (B given as (K, N), A given as (K, M)) is loaded as 8x8 blocks and
// transposed in registers on its way into LDS.  Global loads run CL_GDEPTH steps ahead of the
// matrix cores (register-staged; two LDS stages, one barrier per step), and workgroups are
// renumbered so that each XCD (which owns one L2) works on a compact patch of C.
//
//   CL_M CL_N CL_K            problem size per batch entry (K % (CL_SPLITS*CL_BK) == 0, or unsplit with K % 8 == 0)
//   CL_BM CL_BN CL_BK         workgroup tile;  CL_WM x CL_WN waves, each (BM/WM) x (BN/WN)
//   CL_TRANS_A / CL_TRANS_B   1 when the operand is stored with K as its major / minor axis
//                             opposite to the default (A: (M,K), B: (K,N))
//   CL_BATCH_A CL_BATCH_B     batch counts (grouped broadcast: the larger is the grid's)
//   CL_SPLITS                 split-K factor: partial f32 tiles go to CL_ARG_PACC[split]
//   CL_NORM / CL_GAMMA / CL_EPS   fused RMSNorm of A's rows (see the skinny kernel)
//   CL_GDEPTH                 1 or 2: steps of global loads in flight
//   CL_GROUP_M                row-tiles per patch of the workgroup renumbering

#define GM_THREADS (CL_WM * CL_WN * 64)
#define GM_TM (CL_BM / CL_WM / 16)
#define GM_TN (CL_BN / CL_WN / 16)
#define GM_LD CL_BK                             // LDS row pitch in elements: 128-byte rows, no padding
#define GM_KC (CL_BK / 8)                       // 16-byte chunks along K per tile row
static_assert(CL_BK == 64, "the LDS layout is written for 128-byte tile rows (BK = 64)");
static_assert((GM_TM & (GM_TM - 1)) == 0 && (GM_TN & (GM_TN - 1)) == 0,
              "16-row operand tiles per wave must be a power of two (the swizzle is derived by XOR)");

// Element offset of 16-byte chunk `ch` of tile row `row`.  Rows are 128 bytes; the chunk index is
// XORed with ((row >> 1) ^ (row >> 3)) & 7.  On this hardware a 16-byte-per-lane LDS read is
// served in four phases of lanes {0-3,12-15,20-23,24-27}, {4-11,16-19,28-31}, ... over 64 banks,
// and a 16-byte write in eight phases of 8 consecutive lanes over 32 banks.  With this swizzle
// three access shapes are free of bank conflicts, which no row padding achieves: a matrix-core
// operand read (lane = row l % 16, chunk l / 16), a write of one whole row by 8 consecutive
// lanes, and a write of one chunk of rows r, r + 8, ..., r + 56 by 8 consecutive lanes.
CL_DEVICE int gm_swz(int row) { return ((row >> 1) ^ (row >> 3)) & 7; }
CL_DEVICE int gm_lds_off(int row, int ch) { return row * GM_LD + ((ch ^ gm_swz(row)) << 3); }
#define GM_BATCH (CL_BATCH_A > CL_BATCH_B ? CL_BATCH_A : CL_BATCH_B)
// A contraction length that is not a whole number of BK-wide steps (unsplit, K % 8 == 0): the last
// step's chunks at or past `k_lim` are fetched from the last valid chunk instead and zeroed on
// their way to LDS, in both operands.
#define GM_RAGGED_K ((CL_K / CL_SPLITS) % CL_BK != 0)
static_assert(!GM_RAGGED_K || (CL_SPLITS == 1 && CL_K % 8 == 0), "a ragged last K step needs an unsplit product and 16-byte rows");

// ---- K-minor operand: rows x BK tile, chunk q -> (row q / KC, chunk q % KC) -------------------
template <int ROWS>
struct GmDirect {
  static constexpr int PER = (ROWS * GM_KC + GM_THREADS - 1) / GM_THREADS;
  u32x4 v[PER];
  CL_METHOD void load(const elem_t* __restrict__ base, i64 pitch, int row0, int row_lim, int k0, int k_lim) {
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int q = threadIdx.x + i * GM_THREADS;
      int row = row0 + q / GM_KC;
      row = row < row_lim ? row : row_lim - 1;
      int k = k0 + 8 * (q % GM_KC);
      const bool past = GM_RAGGED_K && k >= k_lim;
      if (GM_RAGGED_K) k = past ? k_lim - 8 : k;
      if (ROWS * GM_KC % GM_THREADS == 0 || q < ROWS * GM_KC) {
        v[i] = ld16(base + (i64)row * pitch + k);
        if (past) v[i] = (u32x4){0u, 0u, 0u, 0u};
      }
    }
  }
  CL_METHOD void store(elem_t* lds) const {
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int q = threadIdx.x + i * GM_THREADS;
      if (ROWS * GM_KC % GM_THREADS == 0 || q < ROWS * GM_KC)
        *reinterpret_cast<u32x4*>(lds + gm_lds_off(q / GM_KC, q % GM_KC)) = v[i];
    }
  }
};

// ---- K-major operand: BK x COLS tile as 8x8 blocks.  Block q -> column block (q % 8) + 8 * (q /
// (8 * KC)), k-block (q / 8) % KC: eight neighbouring lanes read 128 contiguous bytes of one
// global row (one cache line), and their transposed rows go to LDS rows 8 apart at one chunk.
template <int COLS>
struct GmTransposed {
  static constexpr int NB = COLS / 8;
  static constexpr int BLOCKS = GM_KC * NB;
  static constexpr int PER = (BLOCKS + GM_THREADS - 1) / GM_THREADS;
  static_assert(NB % 8 == 0 || NB < 8, "column blocks come in groups of eight");
  static CL_METHOD int cblock(int q) { return NB < 8 ? q % NB : (q & 7) + 8 * (q / (8 * GM_KC)); }
  static CL_METHOD int kblock(int q) { return NB < 8 ? q / NB : (q >> 3) % GM_KC; }
  u32x4 v[PER][8];
  CL_METHOD void load(const elem_t* __restrict__ base, i64 pitch, int col0, int col_lim, int k0, int k_lim) {
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int q = threadIdx.x + i * GM_THREADS;
      if (BLOCKS % GM_THREADS == 0 || q < BLOCKS) {
        int col = col0 + 8 * cblock(q);
        col = col < col_lim - 8 ? col : col_lim - 8;
        int k = k0 + 8 * kblock(q);
        const bool past = GM_RAGGED_K && k >= k_lim;
        if (GM_RAGGED_K) k = past ? k_lim - 8 : k;
        const elem_t* p = base + (i64)k * pitch + col;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          v[i][e] = ld16(p + (i64)e * pitch);
          if (past) v[i][e] = (u32x4){0u, 0u, 0u, 0u};
        }
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
#pragma unroll
        for (int j = 0; j < 8; ++j)
          *reinterpret_cast<u32x4*>(lds + gm_lds_off(8 * cblock(q) + j, kblock(q))) = t[j];
      }
    }
  }
};

// ---- the same operand moved as 4 x 8 half blocks (four k rows of eight columns), for tiles with
// fewer 8x8 blocks than threads: every thread takes part and stages half the registers.  Unit u
// -> column block (u % 8) + 8 * (u / (16 * KC)), k rows 8 * ((u / 16) % KC) + 4 * ((u / 8) % 2).
// Sixteen neighbouring lanes write both 8-byte halves of one chunk of rows 8 apart.
template <int COLS>
struct GmTransposedHalf {
  static constexpr int NB = COLS / 8;
  static constexpr int UNITS = 2 * GM_KC * NB;
  static constexpr int PER = (UNITS + GM_THREADS - 1) / GM_THREADS;
  static_assert(NB % 8 == 0, "column blocks come in groups of eight");
  static CL_METHOD int cblock(int u) { return (u & 7) + 8 * (u / (16 * GM_KC)); }
  static CL_METHOD int kblock(int u) { return (u >> 4) % GM_KC; }
  static CL_METHOD int half(int u) { return (u >> 3) & 1; }
  u32x4 v[PER][4];
  CL_METHOD void load(const elem_t* __restrict__ base, i64 pitch, int col0, int col_lim, int k0, int k_lim) {
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int u = threadIdx.x + i * GM_THREADS;
      if (UNITS % GM_THREADS == 0 || u < UNITS) {
        int col = col0 + 8 * cblock(u);
        col = col < col_lim - 8 ? col : col_lim - 8;
        int k = k0 + 8 * kblock(u);
        const bool past = GM_RAGGED_K && k >= k_lim;
        if (GM_RAGGED_K) k = past ? k_lim - 8 : k;
        const elem_t* p = base + (i64)(k + 4 * half(u)) * pitch + col;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          v[i][e] = ld16(p + (i64)e * pitch);
          if (past) v[i][e] = (u32x4){0u, 0u, 0u, 0u};
        }
      }
    }
  }
  CL_METHOD void store(elem_t* lds) const {
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int u = threadIdx.x + i * GM_THREADS;
      if (UNITS % GM_THREADS == 0 || u < UNITS) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {   // column pair (2q, 2q+1) lives in dword q of every row
          const u32 r0 = v[i][0][q], r1 = v[i][1][q], r2 = v[i][2][q], r3 = v[i][3][q];
          const u32x2 even = {(r0 & 0xffffu) | (r1 << 16), (r2 & 0xffffu) | (r3 << 16)};
          const u32x2 odd = {(r0 >> 16) | (r1 & 0xffff0000u), (r2 >> 16) | (r3 & 0xffff0000u)};
          *reinterpret_cast<u32x2*>(lds + gm_lds_off(8 * cblock(u) + 2 * q, kblock(u)) + 4 * half(u)) = even;
          *reinterpret_cast<u32x2*>(lds + gm_lds_off(8 * cblock(u) + 2 * q + 1, kblock(u)) + 4 * half(u)) = odd;
        }
      }
    }
  }
};

template <int COLS, bool HALF> struct GmPickTransposed { typedef GmTransposed<COLS> type; };
template <int COLS> struct GmPickTransposed<COLS, true> { typedef GmTransposedHalf<COLS> type; };
// half blocks when whole ones would leave threads without work
#define GM_TRANSPOSED(COLS) GmPickTransposed<(COLS), ((COLS) % 64 == 0 && GM_KC * ((COLS) / 8) < GM_THREADS)>::type

#ifndef CL_GDEPTH
#define CL_GDEPTH 1
#endif
#ifndef CL_GROUP_M
#define CL_GROUP_M 4
#endif
#define GM_XCDS 8

// LDS reads issued under the cover of row `i` of 32-wide k block `s` (see GM_COMPUTE).
constexpr int gm_reads_after(int s, int i) {
  int n = 0;
  if (s * GM_TM + i + 2 < 2 * GM_TM) ++n;
  if (s == 0)
    for (int j = 0; j < GM_TN; ++j)
      if (j % GM_TM == i) ++n;
  return n;
}

// The scheduling groups of one step after its leading reads: per row, GM_TN matrix ops and then
// the LDS reads issued under their cover.
template <int S, int I>
CL_DEVICE void gm_sched_rows() {
  __builtin_amdgcn_sched_group_barrier(0x008, GM_TN, 0);
  constexpr int n = gm_reads_after(S, I);
  if constexpr (n > 0) __builtin_amdgcn_sched_group_barrier(0x100, n, 0);
  if constexpr (I + 1 < GM_TM) gm_sched_rows<S, I + 1>();
  else if constexpr (S == 0) gm_sched_rows<1, 0>();
}

#if CL_EMIT_PARTIAL
extern "C" __global__ void __launch_bounds__(GM_THREADS)
CL_PARTIAL_NAME(CL_PARTIAL_PARAMS) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int c = lane & 15, g = lane >> 4;
  const int wm = wave / CL_WN, wn = wave % CL_WN;
  // Workgroups are handed to the XCDs round-robin in launch order.  Renumber them so that the
  // ones an XCD runs at the same time are neighbours in C: launch id L -> the (L / 8)-th tile of
  // XCD (L % 8)'s contiguous share, tiles ordered in patches of CL_GROUP_M row-tiles.
  constexpr int tiles_m = (CL_M + CL_BM - 1) / CL_BM, tiles_n = (CL_N + CL_BN - 1) / CL_BN;
  constexpr int tiles = tiles_m * tiles_n;
  int tile_id = blockIdx.y * tiles_n + blockIdx.x;
  {
    const int xcd = tile_id % GM_XCDS, nth = tile_id / GM_XCDS;
    constexpr int share = tiles / GM_XCDS, extra = tiles % GM_XCDS;
    tile_id = xcd * share + (xcd < extra ? xcd : extra) + nth;
  }
  constexpr int group_m = CL_GROUP_M < tiles_m ? CL_GROUP_M : tiles_m;
  const int band = tile_id / (group_m * tiles_n);
  const int band_rows = (tiles_m - band * group_m) < group_m ? (tiles_m - band * group_m) : group_m;
  const int in_band = tile_id - band * group_m * tiles_n;
  const int m0 = (band * group_m + in_band % band_rows) * CL_BM, n0 = (in_band / band_rows) * CL_BN;
  const int batch = blockIdx.z / CL_SPLITS, split = blockIdx.z % CL_SPLITS;
  constexpr int k_per_split = CL_K / CL_SPLITS;
  const int k_begin = split * k_per_split;
  constexpr int KT = (k_per_split + CL_BK - 1) / CL_BK;
  const int k_lim = k_begin + k_per_split;

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
  typedef GM_TRANSPOSED(CL_BM) LoaderA;
#define GM_LOAD_A(set, kk) set.load(A, CL_M, m0, CL_M, (kk), k_lim)
#else
  typedef GmDirect<CL_BM> LoaderA;
#define GM_LOAD_A(set, kk) set.load(A, CL_K, m0, CL_M, (kk), k_lim)
#endif
#if CL_TRANS_B
  typedef GmDirect<CL_BN> LoaderB;
#define GM_LOAD_B(set, kk) set.load(B, CL_K, n0, CL_N, (kk), k_lim)
#else
  typedef GM_TRANSPOSED(CL_BN) LoaderB;
#define GM_LOAD_B(set, kk) set.load(B, CL_N, n0, CL_N, (kk), k_lim)
#endif
  LoaderA la0;
  LoaderB lb0;
#if CL_GDEPTH > 1
  LoaderA la1;
  LoaderB lb1;
#endif

  f32x4 acc[GM_TM][GM_TN];
#pragma unroll
  for (int i = 0; i < GM_TM; ++i)
#pragma unroll
    for (int j = 0; j < GM_TN; ++j) acc[i][j] = (f32x4){0.f, 0.f, 0.f, 0.f};
  // this lane's operand chunk in the wave's first 16-row tile, k block 0
  const int a_frag = gm_lds_off(wm * (CL_BM / CL_WM) + c, g), b_frag = gm_lds_off(wn * (CL_BN / CL_WN) + c, g);

#if CL_NORM && !CL_TRANS_A
  float ss_local[GmDirect<CL_BM>::PER];
#pragma unroll
  for (int i = 0; i < GmDirect<CL_BM>::PER; ++i) ss_local[i] = 0.f;
  // sum of squares of the raw rows, then gamma folded into the tile on its way to LDS
#define GM_NORM_A(set, kk)                                                          \
  _Pragma("unroll") for (int i = 0; i < GmDirect<CL_BM>::PER; ++i) {               \
    elem8 x = as_elem8(set.v[i]);                                                   \
    _Pragma("unroll") for (int e = 0; e < 8; ++e) {                                \
      const float xf = to_f32(x[e]);                                                \
      ss_local[i] += xf * xf;                                                       \
    }                                                                               \
    GM_GAMMA_A(kk)                                                                  \
    set.v[i] = as_u32x4(x);                                                         \
  }
#if CL_GAMMA
#define GM_GAMMA_A(kk)                                                                              \
  {                                                                                                 \
    const int q = threadIdx.x + i * GM_THREADS;                                                     \
    int gk = (kk) + 8 * (q % GM_KC);                                                                \
    gk = gk < CL_K - 8 ? gk : CL_K - 8;          /* (a chunk past K is zero already) */             \
    elem8 gm = as_elem8(ld16(CL_ARG_GAMMA + gk));                                                   \
    _Pragma("unroll") for (int e = 0; e < 8; ++e) x[e] = to_elem(to_f32(x[e]) * to_f32(gm[e]));    \
  }
#else
#define GM_GAMMA_A(kk)
#endif
#else
#define GM_NORM_A(set, kk)
#endif

  // k offset of step `kt`, clamped to the last step so that prefetches past the end stay in
  // bounds (their data is never stored); unconditional loads keep the wait counts exact
#define GM_KOFF(kt) (k_begin + ((kt) < KT ? (kt) : KT - 1) * CL_BK)

  // Matrix-core work of one step on LDS stage `cur`, software-pipelined: the B fragments of a
  // 32-wide k block stay in registers, the A fragments stream two ahead of their use, and the
  // next k block's B fragments arrive during the first GM_TN rows.  The group barriers pin the
  // order "GM_TN matrix ops, then the reads issued under their cover" so that no LDS latency is
  // waited for with the matrix cores idle.
#define GM_AFRAG(s, i) (*reinterpret_cast<const elem8*>(a_tile + 16 * (i) * GM_LD + (a_frag ^ ((s) * 32) ^ (((2 * (i)) & 7) << 3))))
#define GM_BFRAG(s, j) (*reinterpret_cast<const elem8*>(b_tile + 16 * (j) * GM_LD + (b_frag ^ ((s) * 32) ^ (((2 * (j)) & 7) << 3))))
#define GM_COMPUTE(cur)                                                                                  \
  {                                                                                                      \
    const elem_t* a_tile = As + (cur) * A_STAGE;                                                          \
    const elem_t* b_tile = Bs + (cur) * B_STAGE;                                                          \
    elem8 af[2][GM_TM], bf[2][GM_TN];                                                                     \
    _Pragma("unroll") for (int j = 0; j < GM_TN; ++j) bf[0][j] = GM_BFRAG(0, j);                         \
    af[0][0] = GM_AFRAG(0, 0);                                                                            \
    af[1 / GM_TM][1 % GM_TM] = GM_AFRAG(1 / GM_TM, 1 % GM_TM);                                            \
    _Pragma("unroll") for (int s = 0; s < 2; ++s) {                                                      \
      _Pragma("unroll") for (int i = 0; i < GM_TM; ++i) {                                                \
        /* rows of the MFMA result follow its first operand: feeding B first leaves each lane */         \
        /* with four consecutive columns of one row of C */                                              \
        _Pragma("unroll") for (int j = 0; j < GM_TN; ++j) acc[i][j] = mfma16(bf[s][j], af[s][i], acc[i][j]); \
        /* the A fragments form one sequence over both k blocks, read two ahead of their use */          \
        if (s * GM_TM + i + 2 < 2 * GM_TM)                                                                \
          af[(s * GM_TM + i + 2) / GM_TM][(i + 2) % GM_TM] = GM_AFRAG((s * GM_TM + i + 2) / GM_TM, (i + 2) % GM_TM); \
        if (s == 0) {                                                                                     \
          _Pragma("unroll") for (int j = 0; j < GM_TN; ++j)                                              \
            if (j % GM_TM == i) bf[1][j] = GM_BFRAG(1, j);                                                \
        }                                                                                                 \
      }                                                                                                   \
    }                                                                                                     \
    __builtin_amdgcn_sched_group_barrier(0x100, GM_TN + 2, 0);                                            \
    gm_sched_rows<0, 0>();                                                                                \
  }

  // One step: issue the loads that run CL_GDEPTH steps ahead into (new_a, new_b), work on stage
  // `cur`, then move the oldest staged registers (old_a, old_b: step kt + 1) into the other stage.
  // With two steps in flight the registers of step kt + 1 arrived during the previous step, so
  // they go to LDS first and the writes drain under the matrix ops; with one step in flight the
  // loads need the matrix ops' time to arrive and the writes come last.
#define GM_STORE_NEXT(kt, cur, old_a, old_b)                      \
    if ((kt) + 1 < KT) {                                          \
      GM_NORM_A(old_a, GM_KOFF((kt) + 1))                         \
      old_a.store(As + ((cur) ^ 1) * A_STAGE);                    \
      old_b.store(Bs + ((cur) ^ 1) * B_STAGE);                    \
    }
#if CL_GDEPTH > 1
#define GM_STEP(kt, cur, new_a, new_b, old_a, old_b)              \
  {                                                               \
    GM_LOAD_A(new_a, GM_KOFF((kt) + CL_GDEPTH));     \
    GM_LOAD_B(new_b, GM_KOFF((kt) + CL_GDEPTH));     \
    GM_STORE_NEXT(kt, cur, old_a, old_b)            \
    GM_COMPUTE(cur)                               \
    __syncthreads();                                              \
  }
#else
#define GM_STEP(kt, cur, new_a, new_b, old_a, old_b)              \
  {                                                               \
    GM_LOAD_A(new_a, GM_KOFF((kt) + CL_GDEPTH));     \
    GM_LOAD_B(new_b, GM_KOFF((kt) + CL_GDEPTH));     \
    GM_COMPUTE(cur)                               \
    GM_STORE_NEXT(kt, cur, old_a, old_b)            \
    __syncthreads();                                              \
  }
#endif

  GM_LOAD_A(la0, k_begin);
  GM_LOAD_B(lb0, k_begin);
  GM_NORM_A(la0, k_begin)
  la0.store(As);
  lb0.store(Bs);
#if CL_GDEPTH > 1
  GM_LOAD_A(la1, GM_KOFF(1));
  GM_LOAD_B(lb1, GM_KOFF(1));
#endif
  __syncthreads();

#if CL_GDEPTH > 1
  // register sets alternate: at even steps set 0 receives step kt + 2 while set 1 (step kt + 1)
  // is stored; at odd steps the roles swap
  int kt = 0;
  for (; kt + 1 < KT; kt += 2) {
    GM_STEP(kt, 0, la0, lb0, la1, lb1)
    GM_STEP(kt + 1, 1, la1, lb1, la0, lb0)
  }
  if (kt < KT) GM_STEP(kt, 0, la0, lb0, la1, lb1)
#else
  for (int kt = 0; kt < KT; ++kt) GM_STEP(kt, kt & 1, la0, lb0, la0, lb0)
#endif

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
      if (n0 == 0 && wn == 0 && j == 0 && g == 0) CL_ARG_PSS[((i64)split * GM_BATCH + batch) * CL_M + m] = tot;
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
