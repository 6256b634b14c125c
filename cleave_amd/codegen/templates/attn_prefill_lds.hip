// ---- causal prefill attention (GQA), key tiles shared through LDS ------------------------------
//
// Same operator as attn_prefill.hip (ragged queries; keys through a token table or packed per
// request; keep kv_pos <= kv_len - q_len + q_pos), built for long requests: a workgroup of four
// waves owns 128 query rows of one request and kv head (PL_QT = 128 / group consecutive query
// tokens x the head group; each wave two 16-row tiles) and every 32-key step of K and V is
// loaded once for all of them, global -> LDS directly (16 bytes per lane, table rows looked up per
// lane), as two token-major images in the layout of the MLA kernels:
//   image [D/64][32][64]   64-feature panels, 128-byte key rows, 16-byte chunk ^ (key & 6)
// K is read as the A operand of scores^T = K Q^T with 16-byte reads, V with transposing reads as
// the A operand of out^T += V^T P^T; each operand read feeds both row tiles of the wave.  Three
// stages rotate (two steps of loads in flight), one barrier per step.  The softmax is the exact
// online one (running max per query row, accumulators rescaled only when a max moved), slimmed
// for the vector unit, which is the busiest unit of this kernel: the loop is unrolled over the
// three stages so that LDS addresses are immediates, steps below every row's causal limit run a
// body without mask arithmetic, scale and max subtraction are one multiply-add per score, the
// row maximum crosses the four key groups with two row-swap instructions, and one sum of the
// unrounded weights serves both the normalisation and the lse.
//
// Work items: a new item at every multiple of PL_QT packed query tokens and at every request
// boundary (item t = chunk w + request b for the one pair that overlaps); an item stops at the
// last key any of its rows may see and writes zeros / -inf without reading when it sees none.
//
// CL_DENSE: the same kernel over dense operands Q (units, rows, d), K and V (units, keys, d), every
// row seeing every key (the dense attention family with many query rows per unit): CL_ROWS,
// CL_SKV and CL_SCALE are constants, an item is 128 consecutive rows of one unit, there are no
// row pointers and no lse.
//
// CL_SPLITS > 1 (dense mode): the 32-key steps are dealt out to CL_SPLITS ranges of
// ceil(steps / CL_SPLITS) steps each (the split of attn_decode.hip; the last ranges may be short or
// empty), grid.z = split; a workgroup walks its range only and writes f32 partials (split, row[,
// feature]): the reference point m, the weight sum l against it and the unnormalised values, which
// attn_combine.hip merges by the max-rescale rule (an empty range: m = -huge, l = 0, zeros).  In
// linear mode the partials are plain sums: m = 0 and l = 1 / CL_SPLITS make the same combine add
// them up.
//
// CL_LINEAR (dense mode): no softmax -- out = (q k^T) v, the raw scores times CL_SCALE, rounded to the
// element type, are the weights; no maxima, no reference, no normalisation.
//
// CL_KT (dense mode): the keys are given feature-major, K (units, d, keys) -- the middle operand of a
// chained product (a b) c with b stored (K, N).  A step's K image is then [D/64][64 features][32 keys]
// (64-byte feature rows; the 32-byte halves of a row trade places on rows with feature bit 3 set,
// which spreads the four lane groups of an operand read over the banks), wave w loads features
// 16 w .. 16 w + 15 of every panel, and the score operand (key row, 8 consecutive features) comes
// out of a pair of transposing reads like the value operand does.  CL_SKV must be a multiple of 32.
//
// CL_QNORM / CL_KNORM (QK-norm attention): query / key rows enter the scores RMS-normalised over
// their features, x * rsqrt(mean(x^2) + eps).  Query rows are normalised once when they are loaded.
// Key rows cannot be touched on their way into LDS, so their factors multiply the scores instead:
// the sum of squares of the 16 keys of a score tile is the diagonal of K K^T, which the matrix
// unit makes from the key fragments already in registers (A and B operand are the same
// registers); the lanes on the diagonal take the reciprocal root and the lanes of each score
// fetch the factor of its key.
//
// CL_PF_XCD / CL_PF_REVERSE (default 1) switch the XCD mapping and the walking order.
//
//   CL_HEAD_DIM (multiple of 64)  CL_KV_HEADS  CL_Q_HEADS (group divides 16)  CL_RAGGED
//   run-time: batch, total_q, n_idx (table length / total_kv), num_pages (table form), sm_scale

#ifndef CL_PF_XCD
#define CL_PF_XCD 1
#endif
#ifndef CL_PF_REVERSE
#define CL_PF_REVERSE 1
#endif
#ifndef CL_DENSE
#define CL_DENSE 0
#endif
#ifndef CL_LINEAR
#define CL_LINEAR 0
#endif
#ifndef CL_KT
#define CL_KT 0
#endif
#if CL_KT && (!CL_DENSE || CL_SKV % 32 != 0)
#error "feature-major keys: dense operands, a key count in whole 32-key steps"
#endif
#ifndef CL_QNORM
#define CL_QNORM 0
#endif
#ifndef CL_KNORM
#define CL_KNORM 0
#endif
#if CL_DENSE && !CL_RAGGED
#error "dense operands have consecutive key rows (CL_RAGGED)"
#endif
#if CL_SPLITS > 1 && !CL_DENSE
#error "split keys: dense operands only"
#endif
#define PL_STEP 32
#define PL_GROUP (CL_Q_HEADS / CL_KV_HEADS)
#define PL_ROWS 128
#define PL_QT (PL_ROWS / PL_GROUP)            // query tokens per item
#define PL_KPANELS (CL_HEAD_DIM / 64)         // key width and value width (CL_VDIM) may differ
#define PL_VPANELS (CL_VDIM / 64)
#define PL_PANEL (PL_STEP * 64)               // elements of one 64-feature panel
#define PL_KIMG (PL_KPANELS * PL_PANEL)       // elements of the K image
#define PL_STAGE ((PL_KPANELS + PL_VPANELS) * PL_PANEL)   // K image, then V image
#define PL_STAGES 4
#define PL_KJ (CL_HEAD_DIM / 32)
#define PL_FB (CL_VDIM / 16)
#define PL_UNITS_PER (PL_KPANELS + PL_VPANELS)   // 1 KiB loads per wave and step: its 8-key group of every panel of K and V
static_assert(CL_Q_HEADS % CL_KV_HEADS == 0 && 16 % PL_GROUP == 0, "the head group divides the 16-row query tile");
static_assert(CL_HEAD_DIM % 64 == 0 && CL_HEAD_DIM <= 256 && CL_VDIM % 64 == 0 && CL_VDIM <= 256,
              "key and value widths in whole 64-feature panels");
static_assert(PL_UNITS_PER < 16, "load counter range");

__shared__ __attribute__((aligned(1024))) elem_t pl_tiles[PL_STAGES * PL_STAGE];
#if !CL_RAGGED
__shared__ __attribute__((aligned(256))) int pl_ids[2][4][64];   // table entries on their way in: [step parity][wave][lane]
#endif

typedef short pl_s16x4 __attribute__((ext_vector_type(4)));
typedef short pl_s16x8 __attribute__((ext_vector_type(8)));
typedef __attribute__((address_space(3))) pl_s16x4 pl_lds_s16x4;

CL_DEVICE int pl_swz(int key) { return key & 6; }
CL_DEVICE int pl_clamp(int v, int lo, int hi) { return v < lo ? lo : (v > hi ? hi : v); }

// 16 bytes per lane, global -> LDS (see the MLA kernels): not counted by the compiler, the kernel
// waits for it itself
template <int OFF>
CL_DEVICE void pl_dma16(const void* gptr, unsigned lds_byte) {
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off offset:%2"
               :: "v"(gptr), "s"(__builtin_amdgcn_readfirstlane(lds_byte)), "n"(OFF) : "memory", "m0");
}
// 4 bytes per lane, the same way
CL_DEVICE void pl_dma4(const void* gptr, unsigned lds_byte) {
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %0, off"
               :: "v"(gptr), "s"(__builtin_amdgcn_readfirstlane(lds_byte)) : "memory", "m0");
}

template <int I> struct PlC { static constexpr int value = I; };

// max of x over the four lanes that share lane % 16 (the key groups of one query row): the two
// row-swap instructions exchange 16-lane rows 1<->0', 3<->2' and then 2,3<->0',1' of a register pair
// rows (16 lanes) 1 and 3 of `a` trade places with rows 0 and 2 of `b`
CL_DEVICE void pl_swap_rows16(unsigned& a, unsigned& b) {
  asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 0" : "+v"(a), "+v"(b));
}
CL_DEVICE float pl_max_over_groups(float x) {
  float a = x, b = x;
  asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 0\n\tv_max_f32 %0, %0, %1\n\tv_mov_b32 %1, %0\n\t"
               "s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 0\n\tv_max_f32 %0, %0, %1"
               : "+v"(a), "+v"(b));
  return a;
}

// the largest of three (one instruction, and none of the canonicalising copies fmaxf brings along)
CL_DEVICE float pl_max3(float a, float b, float c) {
  float r;
  asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
  return r;
}
// Row sums of the weights on the matrix unit (a product with a fragment of ones beside the value
// products: the sum of exactly the rounded weights the values are multiplied by) instead of one
// vector add per weight -- where the vector unit is the busier one, i.e. 64-wide heads (measured
// on dense attention over 4096 keys: 151 against 158 us at 64 / 64, 256 against 253 at 128 / 128, 1673
// against 1527 at 192 / 128).  Not where the log-sum-exp is an output: that is held to 1e-3, which the
// rounding of a handful of 16-bit weights would show, so there the unrounded weights are added up.
#ifndef CL_PF_MSUMS
#define CL_PF_MSUMS (CL_HEAD_DIM <= 64 && CL_VDIM <= 64)
#endif
#define PL_MATRIX_SUMS (CL_PF_MSUMS && !CL_EMIT_LSE && !CL_LINEAR)

#if CL_EMIT_PARTIAL
extern "C" __global__ void __launch_bounds__(256, 2)
CL_PARTIAL_NAME(CL_PARTIAL_PARAMS) {
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int c = lane & 15, g = lane >> 4;
  // Workgroups go to the 8 XCDs round-robin in launch order; every XCD has its own L2.  XCD x
  // takes the x-th eighth of the (kv head, item) space (the item axis is padded to a multiple of
  // 8), so the workgroups resident on an XCD are neighbouring items of one kv head and re-read
  // the same keys out of that L2.  Heaviest first: within a request later items see more keys, so
  // every eighth is walked backwards.
  int item, head;
  {
    const int gx = (int)gridDim.x, launch = (int)blockIdx.x + gx * (int)blockIdx.y;
#if CL_PF_XCD
    const int eighth = gx * (int)gridDim.y / 8;
    int lin = (launch % 8) * eighth + launch / 8;
#else
    int lin = launch;
#endif
#if CL_PF_REVERSE
    lin = gx * (int)gridDim.y - 1 - lin;
#endif
    item = lin % gx;
    head = lin / gx;
  }
#if CL_DENSE
  // dense operands: `head` is a unit (batch entry x kv head) with CL_ROWS query rows (its head group
  // x the query positions, all seeing all CL_SKV keys); an item is 128 consecutive rows of them
  const int lo = item * PL_ROWS;
  if (lo >= CL_ROWS) return;                            // (the item axis is padded)
  const int n_rows = CL_ROWS - lo < PL_ROWS ? CL_ROWS - lo : PL_ROWS;
  const int split = CL_SPLITS > 1 ? (int)blockIdx.z : 0;
  constexpr int steps_per_split = ((CL_SKV + 31) / 32 + CL_SPLITS - 1) / CL_SPLITS;
  const int key0 = split * steps_per_split * 32;                     // this split's first key
  int n_keys = CL_SKV - key0 < steps_per_split * 32 ? CL_SKV - key0 : steps_per_split * 32;
  n_keys = n_keys > 0 ? n_keys : 0;
  const int q0 = 0, kv0 = 0, kv_len = n_keys, off = 0, ext = n_keys;
  const float sm_scale = CL_SCALE;
  (void)q0; (void)off;
  auto row_index = [&](int m) __attribute__((always_inline)) { return (i64)head * CL_ROWS + lo + m; };
  auto row_limit = [&](int m) __attribute__((always_inline)) { (void)m; return n_keys - 1; };
#else
  // The request whose items include `item`: the last b with b + qo_indptr[b] / PL_QT <= item, found by
  // all lanes at once (one round trip to memory, which also brings the key row pointers).
  const ClRequest found = cl_find_request(CL_ARG_QINDPTR, batch, total_q, PL_QT, 1, item, lane, CL_ARG_INDPTR, n_idx);
  const int req = found.req, q0 = found.p0, q1 = found.p1, kv0 = found.s0, kv1 = found.s1;
  const int chunk = item - req;
  const int lo = q0 > chunk * PL_QT ? q0 : chunk * PL_QT;
  const int hi = q1 < (chunk + 1) * PL_QT ? q1 : (chunk + 1) * PL_QT;
  if (hi <= lo) return;                                 // an index no (chunk, request) pair maps to
  int kv_len = kv1 - kv0;
  kv_len = kv_len > 0 ? kv_len : 0;
  const int off = kv_len - (q1 - q0);                   // key position of the request's first query row
  const int n_rows = (hi - lo) * PL_GROUP;
  int ext = off + (hi - 1 - q0) + 1;                    // keys the item's last row may see
  ext = ext < kv_len ? ext : kv_len;
  ext = ext > 0 ? ext : 0;

  // output (and query) row of the item's row m, and the last key it may see
  auto row_index = [&](int m) __attribute__((always_inline)) {
    return (i64)(lo + m / PL_GROUP) * CL_Q_HEADS + head * PL_GROUP + m % PL_GROUP;
  };
  auto row_limit = [&](int m) __attribute__((always_inline)) { return off + (lo + m / PL_GROUP - q0); };
#endif

  // this lane's two query rows (column c of each of the wave's score tiles): row index, last key it may see
  bool live[2];
  i64 orow[2];
  int limit[2];
#pragma unroll
  for (int rt = 0; rt < 2; ++rt) {
    const int m = 32 * wave + 16 * rt + c;
    live[rt] = m < n_rows;
    orow[rt] = row_index(live[rt] ? m : 0);
    limit[rt] = live[rt] ? row_limit(m) : -1;
  }

#if CL_SPLITS > 1
  if (ext == 0) {
    // a range past the last key: the partial of nothing
#pragma unroll
    for (int rt = 0; rt < 2; ++rt) {
      if (!live[rt]) continue;
      const i64 prow = (i64)split * CL_TOTAL_ROWS + orow[rt];
      float* dstp = CL_ARG_PO + prow * CL_VDIM + 4 * g;
#pragma unroll
      for (int fb = 0; fb < PL_FB; ++fb) *reinterpret_cast<f32x4*>(dstp + 16 * fb) = (f32x4){0.f, 0.f, 0.f, 0.f};
      if (g == 0) {
        CL_ARG_PM[prow] = CL_LINEAR ? 0.f : CL_NEG_BIG;
        CL_ARG_PL[prow] = CL_LINEAR ? 1.0f / CL_SPLITS : 0.f;
      }
    }
    return;
  }
#else
  if (ext == 0) {
    // no row of the item sees a key: zeros and -inf, nothing to read
#pragma unroll
    for (int rt = 0; rt < 2; ++rt) {
      if (!live[rt]) continue;
      elem_t* dst = CL_ARG_OUT + orow[rt] * CL_VDIM + 16 * (g & 1) + 4 * (g & 2);
#pragma unroll
      for (int fp = 0; fp < PL_FB / 2; ++fp) *reinterpret_cast<u32x4*>(dst + 32 * fp) = (u32x4){0u, 0u, 0u, 0u};
#if CL_EMIT_LSE
      if (g == 0) CL_ARG_LSE[orow[rt]] = CL_NEG_INF;
#endif
    }
    return;
  }
#endif

  // the softmax scale as a positive factor of the raw scores (its sign goes into the Q rows, exactly)
  const float scale2 = fmaxf(fabsf(sm_scale) * 1.4426950408889634f, 1.0e-30f);
  const unsigned q_sign = sm_scale < 0.f ? 0x80008000u : 0u;
#if CL_DENSE
  const i64 krow_bytes = (i64)CL_HEAD_DIM * 2, vrow_bytes = (i64)CL_VDIM * 2;       // K, V: (unit, key, feature)
  // (feature-major keys: a key is a column, the split's first key a byte offset along the rows)
  const char* kbase = reinterpret_cast<const char*>(CL_ARG_K) + (i64)head * CL_SKV * CL_HEAD_DIM * 2 +
                      (i64)key0 * (CL_KT ? 2 : CL_HEAD_DIM * 2);
  const char* vbase = reinterpret_cast<const char*>(CL_ARG_V) + ((i64)head * CL_SKV + key0) * CL_VDIM * 2;
#else
  // K, V: (key row, kv head, feature)
  const i64 krow_bytes = (i64)CL_KV_HEADS * CL_HEAD_DIM * 2, vrow_bytes = (i64)CL_KV_HEADS * CL_VDIM * 2;
  const char* kbase = reinterpret_cast<const char*>(CL_ARG_K) + (i64)head * CL_HEAD_DIM * 2;
  const char* vbase = reinterpret_cast<const char*>(CL_ARG_V) + (i64)head * CL_VDIM * 2;
#endif
  const int n_steps = (ext + PL_STEP - 1) / PL_STEP;
  const unsigned tiles_byte = (unsigned)(size_t)(__attribute__((address_space(3))) elem_t*)pl_tiles;

  // This wave's share of step s (clamped onto the last step: a step past the end reloads the last
  // one into an image nobody reads, so the load counter holds the same number of steps at every
  // wait): key rows 8 wave + lane / 8 of every panel of K and V, the chunk for slot lane % 8.
  // The lane's key row is kv0 + position (packed keys) or its table entry, which `row_of` reads
  // (positions past the item's last key repeat it; ids outside the pool are clamped into it).
  const int my_r = 8 * wave + (lane >> 3);
  auto key_pos = [&](int s) __attribute__((always_inline)) {
    s = s < n_steps - 1 ? s : n_steps - 1;
    const int t = s * PL_STEP + my_r;
    return t < ext - 1 ? t : ext - 1;
  };
  auto row_of = [&](int s) __attribute__((always_inline)) {
#if CL_RAGGED
    return kv0 + key_pos(s);
#else
    return pl_clamp(CL_ARG_INDICES[kv0 + key_pos(s)], 0, num_pages - 1);
#endif
  };
#if !CL_RAGGED
  // In the loop the lane's table entry travels like the tiles do, global -> LDS on the kernel's
  // own load counter, a step ahead of the loads that need it (a load the compiler tracks would
  // make it wait for every load in flight): entry of step s into pl_ids[s & 1][wave][lane].
  const unsigned ids_byte = (unsigned)(size_t)(__attribute__((address_space(3))) int*)&pl_ids[0][0][0];
  auto fetch_id = [&](int s) __attribute__((always_inline)) {
    pl_dma4(CL_ARG_INDICES + kv0 + key_pos(s), ids_byte + (unsigned)(((s & 1) * 4 + wave) * 256));
  };
  auto fetched_row = [&](int s) __attribute__((always_inline)) {
    return pl_clamp(pl_ids[s & 1][wave][lane], 0, num_pages - 1);
  };
#endif
  // load `part` of a step (its K panels, then its V panels) into stage `slot`
  auto issue_part = [&](int row, int slot, auto part_c) __attribute__((always_inline)) {
    constexpr int PART = decltype(part_c)::value;
    constexpr bool IS_K = PART < PL_KPANELS;
    constexpr int P = IS_K ? PART : PART - PL_KPANELS;
    const unsigned group_byte = tiles_byte + (unsigned)(slot * PL_STAGE * 2 + wave * 1024) + (IS_K ? 0 : PL_KIMG * 2);
#if CL_KT
    if constexpr (IS_K) {
      // feature row 64 P + 16 wave + lane / 4 of the (d, keys) matrix, the step's 32 keys as four
      // 16-byte chunks; `row` is the lane's key row of the step, so the step starts at row - my_r
      const int feat = 64 * P + 16 * wave + (lane >> 2);
      const int piece = (lane & 3) ^ ((lane >> 4) & 2);            // halves swapped where feature bit 3 is set
      const char* src = kbase + ((i64)feat * CL_SKV + (row - my_r)) * 2 + 16 * piece;
      pl_dma16<0>(src, group_byte + (unsigned)(P * PL_PANEL * 2));
      return;
    }
#endif
    const int chunk = (lane & 7) ^ pl_swz(my_r);
    const char* src = (IS_K ? kbase + (i64)row * krow_bytes : vbase + (i64)row * vrow_bytes) + 16 * chunk;
    pl_dma16<128 * P>(src, group_byte + (unsigned)(P * PL_PANEL * 2) - 128 * P);
  };
  // the quarter `place` (0..3) of a step's loads: the body spreads them between its matrix work,
  // because a wave stands still while a load waits for the path into the CU
  auto issue_quarter = [&](int row, int slot, auto place_c) __attribute__((always_inline)) {
    constexpr int PLACE = decltype(place_c)::value, LO = PLACE * PL_UNITS_PER / 4, HI = (PLACE + 1) * PL_UNITS_PER / 4;
    if constexpr (HI > LO) issue_part(row, slot, PlC<LO>{});
    if constexpr (HI > LO + 1) issue_part(row, slot, PlC<LO + 1>{});
  };
  auto issue_step = [&](int row, int slot) __attribute__((always_inline)) {
    issue_quarter(row, slot, PlC<0>{});
    issue_quarter(row, slot, PlC<1>{});
    issue_quarter(row, slot, PlC<2>{});
    issue_quarter(row, slot, PlC<3>{});
  };
#define PL_WAITCNT(n) __builtin_amdgcn_s_waitcnt(0x0F70 | ((n) & 15) | (((n) >> 4) << 14))

  {
    const int row0 = row_of(0), row1 = row_of(1), row2 = row_of(2);
    issue_step(row0, 0);
    issue_step(row1, 1);
#if !CL_RAGGED
    fetch_id(3);
#endif
    issue_step(row2, 2);
  }

  // Query rows as the B operand: lane (c, g) holds Q[row][32 j + 8 g .. +8]; padded rows are 0.
  elem8 qf[2][PL_KJ];
#pragma unroll
  for (int rt = 0; rt < 2; ++rt) {
    const elem_t* row = CL_ARG_Q + orow[rt] * CL_HEAD_DIM + 8 * g;
#pragma unroll
    for (int j = 0; j < PL_KJ; ++j) {
      u32x4 raw = ld16(row + 32 * j);
      if (!live[rt]) raw = (u32x4){0u, 0u, 0u, 0u};
      qf[rt][j] = as_elem8(raw ^ q_sign);
    }
#if CL_QNORM
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < PL_KJ; ++j)
#pragma unroll
      for (int i = 0; i < 8; ++i) ss += to_f32(qf[rt][j][i]) * to_f32(qf[rt][j][i]);
    ss += lane_xor(ss, lane, 16);
    ss += lane_xor(ss, lane, 32);
    const float rq = fast_rsqrt(ss * (1.0f / CL_HEAD_DIM) + CL_QNORM_EPS);
#pragma unroll
    for (int j = 0; j < PL_KJ; ++j)
#pragma unroll
      for (int i = 0; i < 8; ++i) qf[rt][j][i] = to_elem(to_f32(qf[rt][j][i]) * rq);
#endif
  }

  float m_run[2] = {CL_NEG_BIG, CL_NEG_BIG};   // running max of the scaled scores (log2 domain), uniform over g
  float l_run[2] = {0.f, 0.f};                 // this lane's share of the sum of the weights
#if PL_MATRIX_SUMS
  f32x4 l_acc[2] = {(f32x4){0.f, 0.f, 0.f, 0.f}, (f32x4){0.f, 0.f, 0.f, 0.f}};   // every component: the sum of row c's weights
  elem8 ones;
#pragma unroll
  for (int i = 0; i < 8; ++i) ones[i] = to_elem(1.0f);
#endif
  f32x4 acc[2][PL_FB];                         // acc[rt][fb][r] = O[row][16 fb + 4 g + r]
#pragma unroll
  for (int rt = 0; rt < 2; ++rt)
#pragma unroll
    for (int fb = 0; fb < PL_FB; ++fb) acc[rt][fb] = (f32x4){0.f, 0.f, 0.f, 0.f};

  // this lane's operand offsets inside an image (elements)
  const int a_lo = c * 64 + ((g ^ pl_swz(c)) << 3);
  const int vtok = 4 * g + (c >> 2);
  const int v_lo = vtok * 64 + (((((c & 3) >> 1)) ^ pl_swz(vtok)) << 3) + 4 * (c & 1);
  // causal limit of the lane's rows relative to its first key slot (slot q of half h is key t0 + 16 h + 4 g + q)
  const int lim_rel[2] = {limit[0] - 4 * g, limit[1] - 4 * g};
  // Steps every key of which every live row of this wave sees need no mask: the wave's first
  // row has the smallest limit (a wave without live rows masks nothing: its rows are not written).
  int n_full = n_steps;
  if (32 * wave < n_rows) {
    const int first_limit = row_limit(32 * wave);
    n_full = first_limit < 0 ? 0 : (first_limit + 1) / PL_STEP;
    n_full = n_full < n_steps ? n_full : n_steps;
  }
  n_full = __builtin_amdgcn_readfirstlane(n_full);

  // scores^T of one step out of the K image in stage SLOT: a 16-byte read per 16-key half and
  // 32-feature block, each feeding the wave's two row tiles
  // (`lo`: the lane's operand offset a_lo / v_lo, or a body's own copy of it, see do_step)
  auto k_frag = [&](auto slot_c, int j, int h, int lo) __attribute__((always_inline)) {
    constexpr int SLOT = decltype(slot_c)::value;
#if CL_KT
    // sixteen lanes address a 4 (feature) x 16 (key) patch, lane c: feature row c / 4, keys 4 (c % 4) .. + 3,
    // and lane c receives the four features of key c; two reads give features 8 g .. 8 g + 7 of block j
    const elem_t* p = pl_tiles + SLOT * PL_STAGE + (j >> 1) * PL_PANEL + (32 * (j & 1) + 8 * g + (c >> 2)) * 32 +
                      16 * (h ^ (g & 1)) + 4 * (c & 3);
    const pl_s16x4 lo4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((pl_lds_s16x4*)(p));
    const pl_s16x4 hi4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((pl_lds_s16x4*)(p + 4 * 32));
    return __builtin_bit_cast(elem8, (pl_s16x8)__builtin_shufflevector(lo4, hi4, 0, 1, 2, 3, 4, 5, 6, 7));
#else
    return *reinterpret_cast<const elem8*>(pl_tiles + SLOT * PL_STAGE + (j >> 1) * PL_PANEL + 16 * h * 64 +
                                           (lo ^ ((4 * (j & 1)) << 3)));
#endif
  };
  // value operand for feature block fb out of the V image in stage SLOT: rows = features
  // 16 fb + (0..15), slots = keys 4 g + (0..3), 16 + 4 g + (0..3)
  auto v_frag = [&](auto slot_c, int fb, int lo) __attribute__((always_inline)) {
    constexpr int SLOT = decltype(slot_c)::value;
    const elem_t* p = pl_tiles + SLOT * PL_STAGE + PL_KIMG + (fb >> 2) * PL_PANEL + (lo ^ (((2 * fb) & 7) << 3));
    const pl_s16x4 lo4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((pl_lds_s16x4*)(p));
    const pl_s16x4 hi4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((pl_lds_s16x4*)(p + 16 * 64));
    return __builtin_bit_cast(elem8, (pl_s16x8)__builtin_shufflevector(lo4, hi4, 0, 1, 2, 3, 4, 5, 6, 7));
  };

#if CL_KNORM
  // Factors of the keys of one step onto its raw scores.  gram[h] = K_h K_h^T for the 16 keys of
  // half h: lane (c, g) holds rows 4 g .. 4 g + 3 of column c, so the lanes with c / 4 == g hold
  // the diagonal entry of key c in register c % 4; score slot q of lane (c, g) belongs to key
  // 4 g + q, whose factor is in lane 20 g + q.
  const int kn_src[4] = {(20 * g + 0) << 2, (20 * g + 1) << 2, (20 * g + 2) << 2, (20 * g + 3) << 2};
  auto scale_by_key_norms = [&](const f32x4 (&gram)[2], f32x4 (&sc)[2][2]) __attribute__((always_inline)) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int sel = c & 3;
      const float d01 = sel & 1 ? gram[h][1] : gram[h][0], d23 = sel & 1 ? gram[h][3] : gram[h][2];
      const float rk = fast_rsqrt((sel & 2 ? d23 : d01) * (1.0f / CL_HEAD_DIM) + CL_KNORM_EPS);
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const float f = __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(kn_src[q], __builtin_bit_cast(int, rk)));
        sc[0][h][q] *= f;
        sc[1][h][q] *= f;
      }
    }
  };
#endif

  // The loop is skewed by one step: body s turns the scores of step s (made in body s - 1) into
  // weights and adds their value product, and between those vector instructions it issues the
  // score products of step s + 1, so that the matrix unit works in the shadow of the softmax.
  f32x4 st[2][2];                              // raw scores^T of the step the next body weighs
#if CL_RAGGED
  PL_WAITCNT(2 * PL_UNITS_PER);
#else
  PL_WAITCNT(2 * PL_UNITS_PER + 1);
#endif
  __syncthreads();
  {
#pragma unroll
    for (int rt = 0; rt < 2; ++rt) st[rt][0] = st[rt][1] = (f32x4){0.f, 0.f, 0.f, 0.f};
#if CL_KNORM
    f32x4 gram[2] = {(f32x4){0.f, 0.f, 0.f, 0.f}, (f32x4){0.f, 0.f, 0.f, 0.f}};
#endif
#pragma unroll
    for (int j = 0; j < PL_KJ; ++j)
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const elem8 a = k_frag(PlC<0>{}, j, h, a_lo);
#pragma unroll
        for (int rt = 0; rt < 2; ++rt) st[rt][h] = mfma16(a, qf[rt][j], st[rt][h]);
#if CL_KNORM
        gram[h] = mfma16(a, a, gram[h]);
#endif
      }
#if CL_KNORM
    scale_by_key_norms(gram, st);
#endif
  }

  // Body of step `step`, whose images are in stage SLOT (compile-time: every LDS address is a
  // register plus an immediate).
  auto do_step = [&](auto slot_c, const int step) __attribute__((always_inline)) {
    constexpr int SLOT = decltype(slot_c)::value;
    // the images of step + 1 have landed when at most the loads of step + 2 are outstanding; the
    // barrier makes that everybody's share and frees the stage step - 1 has left, which the
    // loads of step + 3 fill
    PL_WAITCNT(PL_UNITS_PER);
    __syncthreads();
#if CL_RAGGED
    const int row_ahead = row_of(step + 3);
#else
    // (the entry of step + 3 was asked for a body ago, before the loads the wait above left out)
    const int row_ahead = fetched_row(step + 3);
    fetch_id(step + 4);
#endif
#define PL_ISSUE(place) issue_quarter(row_ahead, (SLOT + 3) % PL_STAGES, PlC<place>{})
    PL_ISSUE(0);

    // operands of this body's matrix work: K of step + 1, V of step (8 + 16 LDS reads).
    // With more than 64 KiB of images (keys wider than 128) the offset field of an LDS instruction no
    // longer reaches every stage from one register per lane pattern, and the dozen address registers
    // the optimiser then kept across the loop were spilled, every reload waiting for the tile loads
    // in flight: each body forms its addresses from a copy of the two lane offsets that the
    // optimiser cannot see through, so none of them lives longer than the body's reads (192-wide
    // keys: 14 spilled registers -> none, 8 % faster; at exactly 64 KiB, 128-wide heads, the same
    // step takes the one spilled register away and costs 4 %: not done there).
    int a_lo_b = a_lo, v_lo_b = v_lo;
    if constexpr (PL_STAGES * PL_STAGE * 2 > 65536) asm volatile("" : "+v"(a_lo_b), "+v"(v_lo_b));
    // (256-wide keys: the fragments of the key image are held half at a time -- the second half is
    // read once the score products of the first have gone out -- or query fragments are spilled)
    constexpr int KH = (PL_KJ > 6 && !CL_KNORM) ? PL_KJ / 2 : PL_KJ;
    elem8 kf[KH][2];
#pragma unroll
    for (int j = 0; j < KH; ++j)
#pragma unroll
      for (int h = 0; h < 2; ++h) kf[j][h] = k_frag(PlC<(SLOT + 1) % PL_STAGES>{}, j, h, a_lo_b);
    elem8 vf[PL_FB];
#pragma unroll
    for (int fb = 0; fb < PL_FB; ++fb) vf[fb] = v_frag(slot_c, fb, v_lo_b);
    __builtin_amdgcn_sched_barrier(0);

    // ---- maxima of the step's scores; raise a row's reference when they pass it by 2^8 -------
    float s[2][8];
#pragma unroll
    for (int rt = 0; rt < 2; ++rt)
#pragma unroll
      for (int i = 0; i < 8; ++i) s[rt][i] = st[rt][i >> 2][i & 3];
    if (step >= n_full) {
      // slot i of the lane is key 32 step + 16 (i / 4) + 4 g + i % 4; a masked slot scores -inf,
      // which a finite reference turns into a weight of exactly 0
#pragma unroll
      for (int rt = 0; rt < 2; ++rt) {
        const int room = lim_rel[rt] - step * PL_STEP;
#pragma unroll
        for (int i = 0; i < 8; ++i) s[rt][i] = 16 * (i >> 2) + (i & 3) <= room ? s[rt][i] : (CL_LINEAR ? 0.f : CL_NEG_INF);
      }
    }
    // (first half of the score products of step + 1 in the shadow of the maxima)
    f32x4 sn[2][2];
#pragma unroll
    for (int rt = 0; rt < 2; ++rt) sn[rt][0] = sn[rt][1] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < PL_KJ / 2; ++j)
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int rt = 0; rt < 2; ++rt) sn[rt][h] = mfma16(kf[j][h], qf[rt][j], sn[rt][h]);
    if constexpr (KH < PL_KJ) {
#pragma unroll
      for (int j = KH; j < PL_KJ; ++j)
#pragma unroll
        for (int h = 0; h < 2; ++h) kf[j - KH][h] = k_frag(PlC<(SLOT + 1) % PL_STAGES>{}, j, h, a_lo_b);
    }
#if !CL_LINEAR
    // (the lane's own eight scores of each row; a row's four lane groups are compared only when
    // some lane passes its row's reference: no row does unless one of its lanes does)
    float mx[2];
#pragma unroll
    for (int rt = 0; rt < 2; ++rt) {
      float v = pl_max3(s[rt][0], s[rt][1], s[rt][2]);
      v = pl_max3(v, s[rt][3], s[rt][4]);
      v = pl_max3(v, s[rt][5], s[rt][6]);
      mx[rt] = pl_max3(v, s[rt][7], s[rt][7]) * scale2;
    }
#pragma unroll
    for (int i = 0; i < 2 * PL_KJ; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);
    }
    if constexpr (KH < PL_KJ) __builtin_amdgcn_sched_group_barrier(0x100, 2 * (PL_KJ - KH), 0);
    if (__builtin_amdgcn_ballot_w64(mx[0] > m_run[0] + 8.0f || mx[1] > m_run[1] + 8.0f)) {
      // cold after the first steps of an item: weights stay below 2^8 against a reference that
      // lags the running maximum by less than 8 (log2 domain)
#pragma unroll
      for (int rt = 0; rt < 2; ++rt) {
        mx[rt] = pl_max_over_groups(mx[rt]);
        const float m_new = mx[rt] > m_run[rt] + 8.0f ? mx[rt] : m_run[rt];
        const float alpha = fast_exp2(m_run[rt] - m_new);
        m_run[rt] = m_new;
        l_run[rt] *= alpha;
#if PL_MATRIX_SUMS
        l_acc[rt] *= alpha;
#endif
#pragma unroll
        for (int fb = 0; fb < PL_FB; ++fb) acc[rt][fb] *= alpha;
      }
    }
#endif  // !CL_LINEAR
    __builtin_amdgcn_sched_barrier(0);
    PL_ISSUE(1);

    // ---- weights of the first row tile beside the rest of the score products -----------------
    elem8 pf[2];
    auto weigh = [&](int rt) __attribute__((always_inline)) {
      float psum = 0.f;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
#if CL_LINEAR
        const float p = s[rt][i] * sm_scale;
#else
        const float p = fast_exp2(__builtin_fmaf(s[rt][i], scale2, -m_run[rt]));
#endif
#if !PL_MATRIX_SUMS
        psum += p;
#endif
        pf[rt][i] = to_elem(p);
      }
      l_run[rt] += psum;
    };
#pragma unroll
    for (int j = PL_KJ / 2; j < PL_KJ; ++j)
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int rt = 0; rt < 2; ++rt) sn[rt][h] = mfma16(kf[KH < PL_KJ ? j - KH : j][h], qf[rt][j], sn[rt][h]);
    weigh(0);
#pragma unroll
    for (int i = 0; i < 2 * PL_KJ; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
    PL_ISSUE(2);

    // ---- weights of the second row tile beside the value product of the first ----------------
#pragma unroll
    for (int fb = 0; fb < PL_FB; ++fb) acc[0][fb] = mfma16(vf[fb], pf[0], acc[0][fb]);
#if PL_MATRIX_SUMS
    l_acc[0] = mfma16(ones, pf[0], l_acc[0]);
#endif
    weigh(1);
#pragma unroll
    for (int i = 0; i < PL_FB; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
    PL_ISSUE(3);

    // ---- value product of the second row tile ------------------------------------------------
#pragma unroll
    for (int fb = 0; fb < PL_FB; ++fb) acc[1][fb] = mfma16(vf[fb], pf[1], acc[1][fb]);
#if PL_MATRIX_SUMS
    l_acc[1] = mfma16(ones, pf[1], l_acc[1]);
#endif
#if CL_KNORM
    // (and the sums of squares of the keys of step + 1, whose factors go onto its scores)
    f32x4 gram[2] = {(f32x4){0.f, 0.f, 0.f, 0.f}, (f32x4){0.f, 0.f, 0.f, 0.f}};
#pragma unroll
    for (int j = 0; j < PL_KJ; ++j)
#pragma unroll
      for (int h = 0; h < 2; ++h) gram[h] = mfma16(kf[j][h], kf[j][h], gram[h]);
    __builtin_amdgcn_sched_barrier(0);
    scale_by_key_norms(gram, sn);
#endif
#pragma unroll
    for (int rt = 0; rt < 2; ++rt)
#pragma unroll
      for (int h = 0; h < 2; ++h) st[rt][h] = sn[rt][h];
  };

  // (where the trip count is a small constant it is kept from the optimiser: a handful of steps
  // would otherwise be laid out in a straight line, and at a 256-wide head that form, short of
  // registers, came back from the compiler with one register of a spilled query fragment not
  // restored; with many steps the counted loop stays a loop and runs 1 - 4 % faster than the
  // one the optimiser cannot count, except at 256-wide heads, where it spills four times as much,
  // and at counts that are not whole turns of the four bodies, where the optimiser peels the rest
  // off and spills sixty registers doing so)
  int trips = n_steps;
#if CL_DENSE
  if constexpr (steps_per_split <= 16 || steps_per_split % 4 != 0 || CL_HEAD_DIM > 192) asm volatile("" : "+s"(trips));
#endif
  for (int step = 0;;) {
    do_step(PlC<0>{}, step);
    if (++step >= trips) break;
    do_step(PlC<1>{}, step);
    if (++step >= trips) break;
    do_step(PlC<2>{}, step);
    if (++step >= trips) break;
    do_step(PlC<3>{}, step);
    if (++step >= trips) break;
  }
  // no load may still be on its way into LDS when the workgroup ends
  PL_WAITCNT(0);

  // ---- each lane writes its rows' features (a row that saw no key: 0 and lse -inf) --------------
  // (row coordinates are worked out again from the lane number, behind a barrier for the
  // optimiser: kept across the loop they would cost registers the loop needs)
  int lane_e = lane;
  asm volatile("" : "+v"(lane_e));
  const int c_e = lane_e & 15, g_e = lane_e >> 4;
#pragma unroll
  for (int rt = 0; rt < 2; ++rt) {
#if PL_MATRIX_SUMS
    const float l = l_acc[rt][0];
#else
    float l = l_run[rt];
    l += lane_xor(l, lane_e, 16);
    l += lane_xor(l, lane_e, 32);
#endif
    const int m = 32 * wave + 16 * rt + c_e;
    if (m >= n_rows) continue;
#if CL_LINEAR
    const float inv = 1.0f;
#else
    const float inv = 1.0f / fmaxf(l, 1.0e-30f);
#endif
    const i64 orow = row_index(m);
#if CL_SPLITS > 1
    // split partials: unnormalised f32 values (16 bytes per lane and block), m and l by the g == 0 lanes
    {
      const i64 prow = (i64)split * CL_TOTAL_ROWS + orow;
      float* dstp = CL_ARG_PO + prow * CL_VDIM + 4 * g_e;
#pragma unroll
      for (int fb = 0; fb < PL_FB; ++fb) *reinterpret_cast<f32x4*>(dstp + 16 * fb) = acc[rt][fb];
      if (g_e == 0) {
#if CL_LINEAR
        CL_ARG_PM[prow] = 0.f;
        CL_ARG_PL[prow] = 1.0f / CL_SPLITS;
#else
        CL_ARG_PM[prow] = m_run[rt];
        CL_ARG_PL[prow] = l;
#endif
      }
      (void)inv;
    }
#else
    // A lane holds features 16 fb + 4 g .. + 3 of its row for every block fb.  Lanes g and g ^ 1
    // trade halves of a pair of blocks (one row swap per register), so that each stores 16
    // contiguous bytes: even g the 8 features from 4 g of the even block, odd g those from
    // 4 (g - 1) of the odd one.
    elem_t* dst = CL_ARG_OUT + orow * CL_VDIM + 16 * (g_e & 1) + 4 * (g_e & 2);
#pragma unroll
    for (int fp = 0; fp < PL_FB / 2; ++fp) {
      elem4 y0, y1;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        y0[r] = to_elem(acc[rt][2 * fp][r] * inv);
        y1[r] = to_elem(acc[rt][2 * fp + 1][r] * inv);
      }
      const u32x2 a = __builtin_bit_cast(u32x2, y0), b = __builtin_bit_cast(u32x2, y1);
      unsigned a0 = a[0], a1 = a[1], b0 = b[0], b1 = b[1];
      pl_swap_rows16(a0, b0);
      pl_swap_rows16(a1, b1);
      *reinterpret_cast<u32x4*>(dst + 32 * fp) = (u32x4){a0, a1, b0, b1};
    }
#if CL_EMIT_LSE
    if (g_e == 0) CL_ARG_LSE[orow] = l > 0.f ? m_run[rt] + fast_log2(l) : CL_NEG_INF;
#endif
#endif
  }
}
#endif  // CL_EMIT_PARTIAL
