// ---- LDS-tiled MFMA matmul with direct global->LDS loads: C[M, N] = A[M, K] * B[K, N] ---------
//
// A workgroup owns a BM x BN tile of C and walks K in steps of 64.  Both operand tiles go from
// global memory straight into LDS (global_load_lds, 16 bytes per lane, no register staging, no
// LDS store instructions); a lane chooses which 16-byte chunk it fetches, so the LDS image can
// be swizzled although a wave's 1 KiB lands in lane order.  Two stages: while the matrix cores
// work on one, the loads of the next step fill the other; one barrier per step.
//
// Tile images in LDS (the 16-byte chunk index of a row is XORed with a function of the row so
// that the operand reads are free of bank conflicts):
//   K-minor operand (A as (M,K), B as (N,K)):  [rows][64]   operand fragment = one ds_read_b128
//   K-major operand (B as (K,N), A as (K,M)):  [64][cols]   operand fragment = two transposing
//       reads (ds_read_b64_tr_b16): within 16 lanes, lane 4a+b receives element b of the 8-byte
//       pieces addressed by lanes a, 4+a, 8+a, 12+a; the sixteen lanes address a 4(k) x 16(col)
//       patch (lane j: row j/4, columns 4 (j%4)..+3), so lane c ends up with four consecutive k
//       of column c.
//
//   CL_M CL_N CL_K  CL_BM CL_BN  CL_WM x CL_WN waves  CL_TRANS_A / CL_TRANS_B  CL_BATCH_A/B
//   CL_SPLITS (split-K: f32 partial tiles to CL_ARG_PACC[split])  CL_GROUP_M (tile order patch)
//
// CL_ROWSUM: out[m] = sum over n of (A * B)[m, n].  A workgroup owns BM rows and walks every
// column tile of B with the same accumulators (the sum over columns needs no per-column result:
// the K steps of all column tiles are one long step sequence), then adds up each row: over the
// lane's accumulators, over the four lane groups, over the waves that share the rows (LDS).
//
// CL_SWIGLU: C = (A * B) .* silu(A * G) with a second weight G (CL_ARG_C) laid out like B.  The
// B tile is made of two halves, columns n0 .. n0 + BN/2 of B and the same columns of G, so a
// workgroup covers BN/2 columns of C; every wave owns the same columns in both halves (half of its
// column fragments each) and multiplies the two accumulators in its epilogue.

// CL_NORM (fused RMSNorm of the rows of A, no learned weight): C = (A * B) scaled per row by
// rsqrt(mean(a^2) + eps).  The scale commutes with the product, so the tile pipeline is untouched:
// every A fragment a wave reads for the matrix cores (each element of its rows exactly once) is also
// squared and summed on the vector unit, in the shadow of the matrix ops, and the epilogue
// multiplies.  Unsplit, A given (M, K).

#define GD_WAVES (CL_WM * CL_WN)
#define GD_THREADS (GD_WAVES * 64)
#define GD_TM (CL_BM / CL_WM / 16)
#define GD_TN (CL_BN / CL_WN / 16)
#define GD_BK 64
#define GD_BATCH (CL_BATCH_A > CL_BATCH_B ? CL_BATCH_A : CL_BATCH_B)
#ifndef CL_GROUP_M
#define CL_GROUP_M 8
#endif
#define GD_XCDS 8
#ifndef CL_SPREAD_LOADS
#define CL_SPREAD_LOADS 0
#endif
#ifndef CL_ASM_LOADS
#define CL_ASM_LOADS 1
#endif
#ifndef CL_SWIGLU
#define CL_SWIGLU 0
#endif
#define GD_OUT_BN (CL_SWIGLU ? CL_BN / 2 : CL_BN)   // columns of C a tile covers
#ifndef CL_ROWSUM
#define CL_ROWSUM 0
#endif
#ifndef CL_TAIL
#define CL_TAIL 0
#endif
#ifndef CL_NORM
#define CL_NORM 0
#endif
#if CL_NORM && (CL_TRANS_A || CL_GAMMA || CL_SPLITS != 1 || CL_SWIGLU || CL_ROWSUM)
#error "the fused norm of the direct-to-LDS matmul: row-major A, no learned weight, unsplit"
#endif
#ifndef CL_ASM_MFMA
#define CL_ASM_MFMA (GD_TM * GD_TN * 4 > 128)   // wave tiles whose accumulators fill a register half
#endif
static_assert(CL_BK == 64, "K steps are 64 wide (128-byte K-minor rows)");
static_assert((GD_TM & (GD_TM - 1)) == 0 && (GD_TN & (GD_TN - 1)) == 0, "wave tiles are powers of two");
static_assert(CL_BM % 16 == 0 && CL_BN % 16 == 0, "tiles are multiples of 16");

typedef __attribute__((address_space(3))) void gd_lds_void;
typedef __attribute__((address_space(1))) const void gd_gbl_void;
typedef short gd_s16x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) gd_s16x4 gd_lds_s16x4;

// operand extents along the non-contraction axis and their LDS images (two stages each)
#define GD_A_ELEMS (CL_BM * GD_BK)
#define GD_B_ELEMS (CL_BN * GD_BK)
__shared__ __attribute__((aligned(1024))) elem_t gd_a0[GD_A_ELEMS];
__shared__ __attribute__((aligned(1024))) elem_t gd_a1[GD_A_ELEMS];
__shared__ __attribute__((aligned(1024))) elem_t gd_b0[GD_B_ELEMS];
__shared__ __attribute__((aligned(1024))) elem_t gd_b1[GD_B_ELEMS];
// CL_STAGES = 3 (tiles of which three images fit LDS): the loads of a step are asked for two steps
// ahead, one slice in front of every row of matrix ops over the whole length of a step, instead
// of all at the top of the step before.  The path from L2 into the compute unit takes a step's
// 64 loads in about a third of the step; asked for all at once, or within half a step, they queue
// and every wave stands still at its loads (measured: 14 % of the kernel with every load an L2
// hit); spread over a whole step they do not, and a load has a whole step more to arrive.
#ifndef CL_STAGES
#define CL_STAGES 2
#endif
#if CL_STAGES == 3
__shared__ __attribute__((aligned(1024))) elem_t gd_a2[GD_A_ELEMS];
__shared__ __attribute__((aligned(1024))) elem_t gd_b2[GD_B_ELEMS];
#if !CL_ASM_LOADS || CL_ROWSUM
#error "three stages: assembly tile loads (the kernel counts its own loads in flight), no row-sum walk"
#endif
#endif
static_assert(CL_STAGES == 2 || CL_STAGES == 3, "two or three LDS stages");

// ---- K-minor image: row r at r * 64, chunk ch at slot ch ^ swz(r) ------------------------------
// (row & 6: measured at the full rate of a linear read for the operand shape, lane = row l % 16, chunk l / 16)
CL_DEVICE int gd_swz_kmin(int row) { return row & 6; }

// ---- K-major image: k row at k * COLS, chunk ch at slot ch ^ f(k); f is even so that the two
// chunks of a 32-byte patch row stay neighbours.  The eight k rows a half wave reads together
// (k = 4 t + i + 8 g', i < 4, g' < 2) get eight different bank positions.
template <int COLS>
CL_DEVICE int gd_swz_kmaj(int k) {
  if (COLS >= 128) return 2 * ((k & 3) | (((k >> 3) & 1) << 2));
  if (COLS == 64) return 2 * (((k >> 1) & 1) | (((k >> 3) & 1) << 1));
  return 0;
}

// One operand of the product: how its tile is fetched and how fragments are read.
//   EXT      tile extent along the operand's own axis (BM for A, BN for B)
//   KMAJOR   stored with K as the major axis
template <int V> struct GdInt { static constexpr int value = V; };
template <bool WIDE> struct GdOffset { typedef u32 type; };
template <> struct GdOffset<true> { typedef i64 type; };
//   DUAL     the tile's second half (rows / columns EXT/2 ..) comes from a second tensor of the
//            same layout, `twin` bytes after the first (the same rows / columns of it)
template <int EXT, bool KMAJOR, bool DUAL = false>
struct GdOperand {
  static constexpr int CPR = EXT / 8;                          // K-major: chunks per k row
  static constexpr int UNITS = EXT * GD_BK * 2 / 1024;         // 1 KiB wave loads per tile
  static constexpr int PER = (UNITS + GD_WAVES - 1) / GD_WAVES;
  static constexpr int SPAN = DUAL ? EXT / 2 : EXT;            // tensor rows / columns under the tile
  // this lane's byte offset (from the tile's first element at k = 0) per unit
  typedef typename GdOffset<DUAL>::type off_t;
  off_t goff[PER];

  // ext0: first row/column of the tile, lim: tensor extent along that axis, pitch: elements
  CL_METHOD void init(int ext0, int lim, int pitch, i64 twin = 0) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int u = wave + i * GD_WAVES;
      if (!KMAJOR) {
        const int r = 8 * u + (lane >> 3);
        const int chunk = (lane & 7) ^ gd_swz_kmin(r);
        int row = ext0 + r % SPAN;
        row = row < lim ? row : lim - 1;                        // rows past the edge repeat the last one
        goff[i] = (off_t)(((row - ext0) * pitch + 8 * chunk) * 2) + (r >= SPAN ? twin : 0);
      } else {
        constexpr int RPU = 64 / CPR > 0 ? 64 / CPR : 1;        // k rows per unit
        const int k = u * RPU + lane / CPR;
        const int chunk = (lane % CPR) ^ gd_swz_kmaj<EXT>(k);
        int col = ext0 + (8 * chunk) % SPAN;
        col = col < lim - 8 ? col : lim - 8;                    // chunks past the edge repeat the last one
        goff[i] = (off_t)((k * pitch + (col - ext0)) * 2) + (8 * chunk >= SPAN ? twin : 0);
      }
    }
  }

  // issue this wave's i-th load of one K step; `base`: the tile's first element of this step (uniform),
  // `lds_byte`: the LDS byte address of the stage's image (a link-time constant: the images are static
  // arrays), `wave_byte`: 1024 * the wave's index in a scalar register.  The LDS target of a load goes to
  // M0 as one scalar add; formed from a generic pointer to the image it cost eight scalar instructions per
  // load (the cast back into the LDS address space checks for the null pointer), 128 a step ahead of the
  // matrix work, which a wave that has its SIMD to itself cannot hide.
  CL_METHOD void issue_unit(int i, const elem_t* base, unsigned lds_byte, unsigned wave_byte) const {
    // (the wave's index out of the scalar `wave_byte`: taken from threadIdx the test below is a
    // divergent branch to the compiler, which then keeps `base` in vector registers inside it and
    // hands the assembly a vector pair where it names a scalar one -- tiles with fewer units than
    // waves did not compile)
    const int u = (int)(wave_byte >> 10) + i * GD_WAVES;
    if (UNITS % GD_WAVES == 0 || u < UNITS) {
      const unsigned m0_value = lds_byte + i * GD_WAVES * 1024 + wave_byte;
#if CL_ASM_LOADS
      // Written as assembly (the default): the tile's first element of the step stays in scalar
      // registers and the lane's 32-bit offset goes in as it is, where the builtin forms a 64-bit
      // address per load in vector registers (two registers and an add each; with the row sums of
      // squares of the fused norm beside a 128-register accumulator tile that is what made the
      // compiler spill the offsets and reload them between the loads, each reload waiting for the
      // loads before it).  The load is then not counted by the compiler; the kernel's own
      // vmcnt(0) at the end of a step covers it.  On the large matmul the two forms measure alike.
      if constexpr (sizeof(off_t) == 4) {
        // (scalar base + 32-bit lane offset: no 64-bit address is formed in vector registers)
        asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                     :: "v"(goff[i]), "s"(base), "s"(m0_value)
                     : "memory", "m0");
      } else {
        asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
                     :: "v"(reinterpret_cast<const char*>(base) + goff[i]), "s"(m0_value)
                     : "memory", "m0");
      }
#else
      __builtin_amdgcn_global_load_lds((gd_gbl_void*)(reinterpret_cast<const char*>(base) + goff[i]),
                                       (gd_lds_void*)(size_t)m0_value, 16, 0, 0);
#endif
    }
  }
  // ... all of them
  CL_METHOD void issue(const elem_t* base, unsigned lds_byte, unsigned wave_byte) const {
#pragma unroll
    for (int i = 0; i < PER; ++i) issue_unit(i, base, lds_byte, wave_byte);
  }
};

// fragment readers --------------------------------------------------------------------------------
// K-minor: `off0` = element offset of (row ext_w + c, chunk g) for the wave's first 16-row tile
CL_DEVICE elem8 gd_read_kmin(const elem_t* tile, int off0, int i, int s) {
  // row 16 i + c has the swizzle of row c; k block s: chunk + 4 s
  return *reinterpret_cast<const elem8*>(tile + 16 * i * 64 + (off0 ^ (s * 32)));
}
// K-major: `off0` = element offset of this lane's 8-byte piece for tile j = 0, k block 0, t = 0
template <int COLS>
CL_DEVICE elem8 gd_read_kmaj(const elem_t* tile, int off0, int j, int s) {
  const gd_lds_s16x4* p0 = (const gd_lds_s16x4*)(tile + ((off0 ^ (j << 4)) + (32 * s) * COLS));
  const gd_lds_s16x4* p1 = (const gd_lds_s16x4*)(tile + ((off0 ^ (j << 4)) + (32 * s + 4) * COLS));
  const gd_s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(const_cast<gd_lds_s16x4*>(p0));
  const gd_s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(const_cast<gd_lds_s16x4*>(p1));
  typedef short s16x8 __attribute__((ext_vector_type(8)));
  const s16x8 v = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  return __builtin_bit_cast(elem8, v);
}

// sum of the squares of a fragment's eight elements onto `sum`
CL_DEVICE float gd_sumsq(elem8 f, float sum) {
#if CL_BF16
#pragma unroll
  for (int e = 0; e < 8; ++e) sum = __builtin_fmaf(to_f32(f[e]), to_f32(f[e]), sum);
#else
  typedef _Float16 gd_h2 __attribute__((ext_vector_type(2)));
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const gd_h2 pair = {f[2 * q], f[2 * q + 1]};
    sum = __builtin_amdgcn_fdot2(pair, pair, sum, false);
  }
#endif
  return sum;
}
#define GD_SUMSQ_VALU (CL_NORM ? (CL_BF16 ? 24 : 4) : 0)   // vector instructions per fragment

// The matrix op.  Through the compiler's builtin, a wave tile whose accumulators fill a whole
// register half (8 x 8 fragments = 256 registers) comes out with the accumulators renamed from op
// to op and copied back inside the loop (three copies per matrix op), and with the load addresses
// spilled and reloaded between the tile loads, each reload waiting for the loads before it: 1900 us
// on the 4096 x 14336 x 4096 product.  Written as assembly with the accumulator tied to one
// accumulation register quadruple every op updates its registers in place (520 us).  The compiler
// does not know such a statement is a matrix op, so what it would insert is written here: two idle
// states ahead of the op (an operand written by a vector instruction just before), and the drain
// between the last matrix op and the first read of an accumulator (gd_acc_drain).  Smaller wave
// tiles compile well through the builtin (measured equal or a little faster), which stays their
// default.
#if CL_ASM_MFMA
#if CL_BF16
#define GD_MFMA_OP "v_mfma_f32_16x16x32_bf16"
#else
#define GD_MFMA_OP "v_mfma_f32_16x16x32_f16"
#endif
#define GD_MFMA(acc, a, b) asm volatile("s_nop 1\n\t" GD_MFMA_OP " %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b))
CL_DEVICE void gd_acc_drain() { asm volatile("s_nop 15\n\ts_nop 15" ::: "memory"); }
CL_DEVICE f32x4 gd_acc_read(const f32x4& acc) {
  float r0, r1, r2, r3;
  asm volatile("v_accvgpr_read_b32 %0, %4\n\tv_accvgpr_read_b32 %1, %5\n\t"
               "v_accvgpr_read_b32 %2, %6\n\tv_accvgpr_read_b32 %3, %7"
               : "=&v"(r0), "=&v"(r1), "=&v"(r2), "=&v"(r3)
               : "a"(acc[0]), "a"(acc[1]), "a"(acc[2]), "a"(acc[3]));
  return (f32x4){r0, r1, r2, r3};
}
#else
#define GD_MFMA(acc, a, b) acc = mfma16(a, b, acc)
CL_DEVICE void gd_acc_drain() {}
CL_DEVICE f32x4 gd_acc_read(const f32x4& acc) { return acc; }
#endif

// LDS read instructions per fragment, and the reads issued under the cover of row `i` of k block
// `s` in GD_COMPUTE
#define GD_A_READS (CL_TRANS_A ? 2 : 1)
#define GD_B_READS (CL_TRANS_B ? 1 : 2)
constexpr int gd_reads_after(int TM, int s, int i) {
  int n = 0;
  if (s * TM + i + 2 < 2 * TM) n += GD_A_READS;
  if (s == 0)
    for (int j = 0; j < GD_TN; ++j)
      if (j % TM == i) n += GD_B_READS;
  return n;
}
template <int TM, int S, int I>
CL_DEVICE void gd_sched_rows() {
  __builtin_amdgcn_sched_group_barrier(0x008, GD_TN, 0);
  if constexpr (GD_SUMSQ_VALU > 0) __builtin_amdgcn_sched_group_barrier(0x002, GD_SUMSQ_VALU, 0);
  constexpr int n = gd_reads_after(TM, S, I);
  if constexpr (n > 0) __builtin_amdgcn_sched_group_barrier(0x100, n, 0);
  if constexpr (I + 1 < TM) gd_sched_rows<TM, S, I + 1>();
  else if constexpr (S == 0) gd_sched_rows<TM, 1, 0>();
}

#if CL_EMIT_PARTIAL
extern "C" __global__ void __launch_bounds__(GD_THREADS)
CL_PARTIAL_NAME(CL_PARTIAL_PARAMS) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int c = lane & 15, g = lane >> 4;
  const int wm = wave / CL_WN, wn = wave % CL_WN;
  const unsigned wave_byte = (unsigned)__builtin_amdgcn_readfirstlane(wave) * 1024u;   // scalar: part of every load's LDS target
  // Workgroups are handed to the XCDs round-robin in launch order.  Renumber them so that the
  // ones an XCD runs at the same time are neighbours in C: launch id L -> the (L / 8)-th tile of
  // XCD (L % 8)'s contiguous share, tiles ordered in patches of CL_GROUP_M row-tiles.
  constexpr int tiles_m = (CL_M + CL_BM - 1) / CL_BM, tiles_n = CL_ROWSUM ? 1 : (CL_N + GD_OUT_BN - 1) / GD_OUT_BN;
  constexpr int tiles = tiles_m * tiles_n;
  // CL_TAIL: the last CL_TAIL tiles (the partly filled final round of a launch that does not divide
  // among the compute units) are each run as two workgroups of half the rows, so that the round
  // keeps twice as many compute units busy for half as long.  The grid is then one-dimensional:
  // the whole tiles first, two workgroups per tail tile after them, the halves of a tile on one XCD.
  constexpr int whole = tiles - CL_TAIL;
  int tile_id = CL_TAIL ? blockIdx.x : blockIdx.y * tiles_n + blockIdx.x;
  int half = -1;
  if (tile_id < whole) {
    const int xcd = tile_id % GD_XCDS, nth = tile_id / GD_XCDS;
    constexpr int share = whole / GD_XCDS, extra = whole % GD_XCDS;
    tile_id = xcd * share + (xcd < extra ? xcd : extra) + nth;
  } else {
    const int t = tile_id - whole;
    if (CL_TAIL % GD_XCDS == 0) {
      const int xcd = t % GD_XCDS, nth = t / GD_XCDS;
      tile_id = whole + (nth >> 1) * GD_XCDS + xcd;
      half = nth & 1;
    } else {
      tile_id = whole + (t >> 1);
      half = t & 1;
    }
  }
  constexpr int group_m = CL_GROUP_M < tiles_m ? CL_GROUP_M : tiles_m;
  const int band = tile_id / (group_m * tiles_n);
  const int band_rows = (tiles_m - band * group_m) < group_m ? (tiles_m - band * group_m) : group_m;
  const int in_band = tile_id - band * group_m * tiles_n;
  const int tile_m0 = (band * group_m + in_band % band_rows) * CL_BM, n0 = (in_band / band_rows) * GD_OUT_BN;
  const int batch = blockIdx.z / CL_SPLITS, split = blockIdx.z % CL_SPLITS;
  constexpr int k_per_split = CL_K / CL_SPLITS;
  const int k_begin = split * k_per_split;
  constexpr int KT_K = k_per_split / GD_BK;                     // steps along K
  constexpr int KT = KT_K * (CL_ROWSUM ? CL_N / CL_BN : 1);     // ... times the column tiles one workgroup walks
#if CL_ROWSUM
  static_assert(CL_N % CL_BN == 0 && CL_SPLITS == 1 && GD_BATCH == 1, "row sums walk whole column tiles, unsplit");
#endif

  const elem_t* A = CL_ARG_A + (i64)(batch / (GD_BATCH / CL_BATCH_A)) * CL_M * CL_K;
  const elem_t* B = CL_ARG_B + (i64)(batch / (GD_BATCH / CL_BATCH_B)) * CL_K * CL_N;

  // The rest of the kernel for a workgroup that owns BM rows from m0 (BM = CL_BM, or half of it for
  // a tail half): TM row fragments per wave.
  auto body = [&](auto bm_tag, const int m0) {
  constexpr int BM = decltype(bm_tag)::value;
  constexpr int TM = BM / CL_WM / 16;
  static_assert(TM >= 1 && (TM & (TM - 1)) == 0, "wave tiles are powers of two");
  // ---- operand movers: tile origin at K step 0 and the uniform advance per step ---------------
  GdOperand<BM, CL_TRANS_A != 0> opa;
  GdOperand<CL_BN, CL_TRANS_B == 0, CL_SWIGLU != 0> opb;
#if CL_SWIGLU
  const i64 b_twin = reinterpret_cast<const char*>(CL_ARG_C) - reinterpret_cast<const char*>(CL_ARG_B);
#else
  const i64 b_twin = 0;
#endif
#if CL_TRANS_A
  opa.init(m0, CL_M, CL_M);                                   // A stored (K, M)
  const elem_t* a_base = A + (i64)k_begin * CL_M + m0;
  constexpr i64 a_step = (i64)GD_BK * CL_M;
#else
  opa.init(m0, CL_M, CL_K);                                   // A stored (M, K)
  const elem_t* a_base = A + (i64)m0 * CL_K + k_begin;
  constexpr i64 a_step = GD_BK;
#endif
#if CL_TRANS_B
  opb.init(n0, CL_N, CL_K, b_twin);                           // B stored (N, K)
  const elem_t* b_base = B + (i64)n0 * CL_K + k_begin;
  constexpr i64 b_step = GD_BK;
#else
  opb.init(n0, CL_N, CL_N, b_twin);                           // B stored (K, N)
  const elem_t* b_base = B + (i64)k_begin * CL_N + n0;
  constexpr i64 b_step = (i64)GD_BK * CL_N;
#endif

  // ---- this lane's fragment offsets -------------------------------------------------------------
  // wave origin inside the tile (SwiGLU: inside each half of the B tile; fragments j < TN/2 come
  // from the first half, the others from the same columns of the second)
  const int am = wm * (BM / CL_WM), bn = wn * (GD_OUT_BN / CL_WN);
#if CL_SWIGLU
#define GD_BSEL(j, x, y) ((j) < GD_TN / 2 ? (x) : (y))
#define GD_BJ(j) ((j) % (GD_TN / 2))
#else
#define GD_BSEL(j, x, y) (x)
#define GD_BJ(j) (j)
#endif
#if CL_TRANS_A
  const int a_f = gd_swz_kmaj<BM>(8 * g + (c >> 2));
  const int a_off = (8 * g + (c >> 2)) * BM + 8 * (((am / 8) ^ a_f) + ((c & 3) >> 1)) + 4 * (c & 1);
#define GD_AFRAG(tile, i, s) gd_read_kmaj<BM>(tile, a_off, i, s)
#else
  const int a_off = (am + c) * 64 + ((g ^ gd_swz_kmin(am + c)) << 3);
#define GD_AFRAG(tile, i, s) gd_read_kmin(tile, a_off, i, s)
#endif
#if CL_TRANS_B
  const int b_off = (bn + c) * 64 + ((g ^ gd_swz_kmin(bn + c)) << 3);
  const int b_off2 = b_off + (CL_BN / 2) * 64;                  // (BN/2 is a multiple of 8: same swizzle)
#define GD_BFRAG(tile, j, s) gd_read_kmin(tile, GD_BSEL(j, b_off, b_off2), GD_BJ(j), s)
#else
  const int b_f = gd_swz_kmaj<CL_BN>(8 * g + (c >> 2));
  const int b_off = (8 * g + (c >> 2)) * CL_BN + 8 * (((bn / 8) ^ b_f) + ((c & 3) >> 1)) + 4 * (c & 1);
  const int b_off2 = (8 * g + (c >> 2)) * CL_BN + 8 * ((((CL_BN / 2 + bn) / 8) ^ b_f) + ((c & 3) >> 1)) + 4 * (c & 1);
#define GD_BFRAG(tile, j, s) gd_read_kmaj<CL_BN>(tile, GD_BSEL(j, b_off, b_off2), GD_BJ(j), s)
#endif

  f32x4 acc[TM][GD_TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < GD_TN; ++j) acc[i][j] = (f32x4){0.f, 0.f, 0.f, 0.f};
#if CL_NORM
  float ss[TM];        // this lane's share of the sum of squares of row am + 16 i + c (k chunks g, g + 4 of every step)
#pragma unroll
  for (int i = 0; i < TM; ++i) ss[i] = 0.f;
#define GD_SUMSQ(i, frag) ss[i] = gd_sumsq(frag, ss[i]);
#else
#define GD_SUMSQ(i, frag)
#endif

  // Matrix-core work of one step on one stage, software-pipelined: the B fragments of a 32-wide
  // k block stay in registers, the A fragments stream two ahead of their use, and the next k
  // block's B fragments arrive spread over the rows of the current one.  Rows of the MFMA result
  // follow its first operand, so feeding B first leaves each lane with four consecutive columns
  // of one row of C.  The group barriers pin the order "GD_TN matrix ops, then the reads issued
  // under their cover" so that no LDS latency is waited for with the matrix cores idle.
#define GD_COMPUTE(a_tile, b_tile, NEXT)                                                            \
  {                                                                                                 \
    elem8 af[2][TM], bf[2][GD_TN];                                                               \
    _Pragma("unroll") for (int j = 0; j < GD_TN; ++j) bf[0][j] = GD_BFRAG(b_tile, j, 0);           \
    af[0][0] = GD_AFRAG(a_tile, 0, 0);                                                              \
    af[1 / TM][1 % TM] = GD_AFRAG(a_tile, 1 % TM, 1 / TM);                              \
    _Pragma("unroll") for (int s = 0; s < 2; ++s) {                                                \
      _Pragma("unroll") for (int i = 0; i < TM; ++i) {                                          \
        NEXT(s * TM + i)                                                                         \
        _Pragma("unroll") for (int j = 0; j < GD_TN; ++j) GD_MFMA(acc[i][j], bf[s][j], af[s][i]);              \
        GD_SUMSQ(i, af[s][i])                                                                       \
        if (s * TM + i + 2 < 2 * TM)                                                          \
          af[(s * TM + i + 2) / TM][(i + 2) % TM] =                                        \
              GD_AFRAG(a_tile, (i + 2) % TM, (s * TM + i + 2) / TM);                       \
        if (s == 0) {                                                                               \
          _Pragma("unroll") for (int j = 0; j < GD_TN; ++j)                                        \
            if (j % TM == i) bf[1][j] = GD_BFRAG(b_tile, j, 1);                                  \
        }                                                                                           \
        GD_ROW_END()                                                                                \
      }                                                                                             \
    }                                                                                               \
    GD_STEP_SCHED()                                                                                 \
  }
#if CL_SPREAD_LOADS || CL_ASM_MFMA || CL_STAGES == 3
// every row of matrix ops closes with a scheduling barrier: the order of the source (this row's
// loads of the next step, its matrix ops, the fragment reads for two rows on) is the order of the
// instruction stream
#define GD_ROW_END() __builtin_amdgcn_sched_barrier(0);
#define GD_STEP_SCHED()
#else
#define GD_ROW_END()
#define GD_STEP_SCHED()                                                                             \
    __builtin_amdgcn_sched_group_barrier(0x100, GD_B_READS * GD_TN + 2 * GD_A_READS, 0);            \
    gd_sched_rows<TM, 0, 0>();
#endif
  // everything this wave loaded has landed; after the barrier, everything every wave loaded
#define GD_STEP_END()                           \
  __builtin_amdgcn_s_waitcnt(0x0F70);           \
  __syncthreads();
  // The loads of the next step.  A wave that issues a load while the path from L2 into the
  // compute unit (64 bytes per clock) is busy stands still, matrix ops and all; every wave
  // issuing its whole share at the top of a step stops the matrix cores for the length of the
  // transfer.  CL_SPREAD_LOADS: row r of a step's matrix work is preceded by the r-th slice of
  // the wave's loads instead (measured: no faster on the large matmul; off by default).
#if CL_ROWSUM
#define GD_A_AT(kt) (a_base + (i64)((kt) % KT_K) * a_step)
#define GD_B_AT(kt) (b_base + (i64)((kt) % KT_K) * b_step + (i64)((kt) / KT_K) * (CL_TRANS_B ? (i64)CL_BN * CL_K : (i64)CL_BN))
#else
#define GD_A_AT(kt) (a_base + (i64)(kt) * a_step)
#define GD_B_AT(kt) (b_base + (i64)(kt) * b_step)
#endif
#define GD_LDS_BYTE(image) ((unsigned)(size_t)(__attribute__((address_space(3))) elem_t*)(image))
#define GD_ISSUE(kt, a_lds, b_lds)                              \
  opa.issue(GD_A_AT(kt), GD_LDS_BYTE(a_lds), wave_byte);        \
  opb.issue(GD_B_AT(kt), GD_LDS_BYTE(b_lds), wave_byte);        \
  __builtin_amdgcn_sched_barrier(0);
#define GD_ISSUE_SLICE(r, kt, a_lds, b_lds)                                                         \
  {                                                                                                 \
    constexpr int ua_ = decltype(opa)::PER, ub_ = decltype(opb)::PER;                               \
    constexpr int per_row_ = (ua_ + ub_ + 2 * TM - 1) / (2 * TM);                             \
    _Pragma("unroll") for (int q_ = (r) * per_row_; q_ < ((r) + 1) * per_row_; ++q_) {             \
      if (q_ < ua_) opa.issue_unit(q_, GD_A_AT(kt), GD_LDS_BYTE(a_lds), wave_byte);                 \
      else if (q_ < ua_ + ub_) opb.issue_unit(q_ - ua_, GD_B_AT(kt), GD_LDS_BYTE(b_lds), wave_byte); \
    }                                                                                               \
  }
#define GD_NO_NEXT(r)

  // Two steps per trip, one on each stage, with no branch inside: the loads issued in the second
  // half are clamped onto the last step (for an even step count the final trip fetches that step
  // once more into the idle stage, which nobody reads).
#if CL_STAGES == 3
  {
    constexpr int per_step_ = decltype(opa)::PER + decltype(opb)::PER;     // loads per wave and step
    static_assert(decltype(opa)::UNITS % GD_WAVES == 0 && decltype(opb)::UNITS % GD_WAVES == 0 && per_step_ < 32,
                  "three stages: every wave issues the same number of loads per step (the wait counts them)");
    // at most the loads this wave asked for during the step just done (those of two steps on) are
    // still on their way: the next step's images have landed; after the barrier, everybody's
#define GD_STEP_END3()                                                                              \
    __builtin_amdgcn_s_waitcnt(0x0F70 | (per_step_ & 15) | ((per_step_ >> 4) << 14));               \
    __syncthreads();
#define GD_AHEAD(kt) ((kt) + 2 < KT ? (kt) + 2 : KT - 1)
#define GD_NEXT_S2(r) GD_ISSUE_SLICE(r, GD_AHEAD(kt), gd_a2, gd_b2)
#define GD_NEXT_S0(r) GD_ISSUE_SLICE(r, GD_AHEAD(kt), gd_a0, gd_b0)
#define GD_NEXT_S1(r) GD_ISSUE_SLICE(r, GD_AHEAD(kt), gd_a1, gd_b1)
    GD_ISSUE(0, gd_a0, gd_b0)
    GD_ISSUE((1 < KT ? 1 : KT - 1), gd_a1, gd_b1)
    GD_STEP_END3()
    // (past the last step the loads are clamped onto it and go into the stage left a step ago,
    // which nobody reads again: every step issues the same number of loads)
    for (int kt = 0;;) {
      GD_COMPUTE(gd_a0, gd_b0, GD_NEXT_S2)
      GD_STEP_END3()
      if (++kt >= KT) break;
      GD_COMPUTE(gd_a1, gd_b1, GD_NEXT_S0)
      GD_STEP_END3()
      if (++kt >= KT) break;
      GD_COMPUTE(gd_a2, gd_b2, GD_NEXT_S1)
      GD_STEP_END3()
      if (++kt >= KT) break;
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);          // no load may still be on its way into LDS past this point
  }
#else
  GD_ISSUE(0, gd_a0, gd_b0)
  GD_STEP_END()
#if CL_SPREAD_LOADS
#define GD_NEXT_1(r) GD_ISSUE_SLICE(r, kt + 1, gd_a1, gd_b1)
#define GD_NEXT_0(r) GD_ISSUE_SLICE(r, (kt + 2 < KT ? kt + 2 : KT - 1), gd_a0, gd_b0)
  for (int kt = 0; kt + 1 < KT; kt += 2) {
    GD_COMPUTE(gd_a0, gd_b0, GD_NEXT_1)
    GD_STEP_END()
    GD_COMPUTE(gd_a1, gd_b1, GD_NEXT_0)
    GD_STEP_END()
  }
#else
  for (int kt = 0; kt + 1 < KT; kt += 2) {
    GD_ISSUE(kt + 1, gd_a1, gd_b1)
    GD_COMPUTE(gd_a0, gd_b0, GD_NO_NEXT)
    GD_STEP_END()
    GD_ISSUE((kt + 2 < KT ? kt + 2 : KT - 1), gd_a0, gd_b0)
    GD_COMPUTE(gd_a1, gd_b1, GD_NO_NEXT)
    GD_STEP_END()
  }
#endif
  if constexpr (KT % 2 == 1) GD_COMPUTE(gd_a0, gd_b0, GD_NO_NEXT)     // an odd number of steps ends on stage 0
#endif  // CL_STAGES

  // ---- epilogue: acc[i][j][r] = C[m0 + am + 16 i + c][n0 + bn + 16 j + 4 g + r] ----------------
  gd_acc_drain();
#if CL_ROWSUM
  {
    __syncthreads();                                  // every wave is done with the tile images
    float* red = reinterpret_cast<float*>(gd_b0);     // [BM][WN]
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      float sum = 0.f;
#pragma unroll
      for (int j = 0; j < GD_TN; ++j) {
        const f32x4 v = gd_acc_read(acc[i][j]);
        sum += (v[0] + v[1]) + (v[2] + v[3]);
      }
      sum += lane_xor(sum, lane, 16);
      sum += lane_xor(sum, lane, 32);
      if (g == 0) red[(am + 16 * i + c) * CL_WN + wn] = sum;
    }
    __syncthreads();
    for (int r = threadIdx.x; r < BM; r += GD_THREADS) {
      if (m0 + r >= CL_M) break;
      float sum = 0.f;
#pragma unroll
      for (int w = 0; w < CL_WN; ++w) sum += red[r * CL_WN + w];
      CL_ARG_OUT[m0 + r] = to_elem(sum);
    }
    return;
  }
#endif
#if CL_NORM
  float row_scale[TM];
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    float t = ss[i];
    t += lane_xor(t, lane, 16);
    t += lane_xor(t, lane, 32);
    row_scale[i] = fast_rsqrt(t * (1.0f / CL_K) + CL_EPS);
  }
#endif
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int m = m0 + am + 16 * i + c;
    if (m >= CL_M) continue;
#if CL_SWIGLU
#pragma unroll
    for (int j = 0; j < GD_TN / 2; ++j) {
      const int n = n0 + bn + 16 * j + 4 * g;
      if (n >= CL_N) continue;
      elem4 y;
      const f32x4 up = gd_acc_read(acc[i][j]), gates = gd_acc_read(acc[i][j + GD_TN / 2]);
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float gate = gates[r];
        y[r] = to_elem(up[r] * gate / (1.0f + __expf(-gate)));
      }
      *reinterpret_cast<elem4*>(CL_ARG_OUT + (i64)m * CL_N + n) = y;
    }
#else
#pragma unroll
    for (int j = 0; j < GD_TN; ++j) {
      const int n = n0 + bn + 16 * j + 4 * g;
      if (n >= CL_N) continue;
      const f32x4 v = gd_acc_read(acc[i][j]);
#if CL_SPLITS > 1
      *reinterpret_cast<f32x4*>(CL_ARG_PACC + (((i64)split * GD_BATCH + batch) * CL_M + m) * CL_N + n) = v;
#else
      elem4 y;
#pragma unroll
#if CL_NORM
      for (int r = 0; r < 4; ++r) y[r] = to_elem(v[r] * row_scale[i]);
#else
      for (int r = 0; r < 4; ++r) y[r] = to_elem(v[r]);
#endif
      *reinterpret_cast<elem4*>(CL_ARG_OUT + ((i64)batch * CL_M + m) * CL_N + n) = y;
#endif
    }
#endif  // CL_SWIGLU
  }
  };
#if CL_TAIL
  static_assert(!CL_ROWSUM && !CL_TRANS_A && GD_BATCH == 1 && CL_SPLITS == 1, "the tail split halves row-major A tiles of an unsplit, unbatched product");
  if (half >= 0) {
    body(GdInt<CL_BM / 2>{}, tile_m0 + half * (CL_BM / 2));
    return;
  }
#endif
  body(GdInt<CL_BM>{}, tile_m0);
}
#endif  // CL_EMIT_PARTIAL
