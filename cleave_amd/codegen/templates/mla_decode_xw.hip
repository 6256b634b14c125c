// ---- MLA decode, 64 heads per workgroup, the two products shared out over the waves two ways --
//
//   out = softmax((q kv^T + q_pe k_pe^T) * scale) kv          latent kv shared by all heads
//
// LDS -> register bandwidth (about 128 bytes per clock and compute unit) bounds this operator
// when every wave reads the whole step image for both products.  Here the four waves of a
// workgroup read as little of it as the matrix-op shapes allow:
//   score product   wave (th, hh) takes the 16 tokens of half th of a 32-token step against the
//                   32 heads of half hh: one 16-byte operand read feeds two matrix ops;
//   value product   wave w takes all 64 heads against features [w CKV/4, (w+1) CKV/4): one pair of
//                   transposing reads feeds four matrix ops.
// The softmax weights cross between the two roles through a small LDS buffer (element type, in
// the operand order of the value product).  The products are skewed by one step: an iteration
// computes the scores of step s+1 and the value product of step s, which are independent, so
// the matrix pipe always has work and the softmax arithmetic sits in its shadow; one barrier
// per step publishes the weights of step s+1 and the image of step s+2 together.
//
// The step image is the token-major one: [D/64][32][64] with the 16-byte chunk index of a row
// XORed with (token & 6), loaded global -> LDS directly (16 bytes per lane), four images
// rotating: two in the matrix cores, two in flight.  The Q rows of the workgroup's heads come in
// the same way (two images, rows = heads) before the first step, are taken into registers and
// their slots handed to steps 2 and 3.
//
// Softmax reference point: fixed per head, raised only when a score exceeds it by more than 8
// (log2 domain).  A wave that sees such a score raises a flag beside the weights; after the
// barrier every wave finds the flag, and the workgroup takes the cold path together: new
// reference = largest candidate, accumulators rescaled, the step's weights recomputed from
// the kept scores.  The first step enters that path with the reference at -huge.
//
//   CL_HEADS (multiple of 64)  CL_CKV (multiple of 256)  CL_KPE (multiple of 64)  CL_SKV
//   CL_SPLITS  CL_BATCH  CL_SCALE_LOG2E  CL_PO_ELEM (as in the one-wave-per-head-set kernel)

#ifndef CL_PO_ELEM
#define CL_PO_ELEM 0
#endif
#define MX_STEP 32
#define MX_D (CL_CKV + CL_KPE)
#define MX_THREADS 256
#define MX_HEADS 64                           // heads per workgroup
#define MX_PANEL (MX_STEP * 64)               // elements of one 64-feature panel of the image
#define MX_PANELS (MX_D / 64)
#define MX_LAT_PANELS (CL_CKV / 64)
#define MX_TILE (MX_PANELS * MX_PANEL)        // elements of one LDS image
#define MX_KJ (MX_D / 32)                     // score matrix ops per 16 tokens and 16 heads
#define MX_FBW (CL_CKV / 64)                  // 16-feature blocks of the value product per wave
#define MX_STAGES 4
#define MX_AHEAD 3                            // steps whose loads have been issued beyond the one in the value product
#define MX_UNITS_PER MX_PANELS                // 1 KiB loads per wave and step (one 8-token group of every panel)
#define MX_RESCALE_STEP 8.0f
#define MX_HEAD_GROUPS (CL_HEADS / MX_HEADS)
#ifndef CL_QA
#define CL_QA MX_KJ
#endif
#define MX_QA (CL_QA < MX_KJ ? CL_QA : MX_KJ) // Q fragments per head tile pinned to the accumulation registers
static_assert(CL_HEADS % MX_HEADS == 0, "64 heads per workgroup");
static_assert(CL_CKV % 256 == 0 && CL_KPE % 64 == 0, "a wave's value features are whole 64-feature panels");
static_assert(CL_SCALE_LOG2E > 0.f, "the largest raw score must be the largest scaled one");
static_assert(2 * MX_UNITS_PER < 64, "load counter range");
static_assert(MX_KJ % 2 == 0, "score contraction in pairs of 32-feature blocks");
constexpr bool MX_RAGGED = CL_SKV % MX_STEP != 0;   // the last step has tokens past the end

__shared__ __attribute__((aligned(1024))) elem_t mx_tiles[MX_STAGES * MX_TILE];
__shared__ __attribute__((aligned(16))) elem_t mx_p[2][MX_HEADS][MX_STEP];   // weights: [head][operand slot]
__shared__ float mx_m[MX_HEADS];              // reference point per head (log2 domain)
__shared__ float mx_cand[2][MX_HEADS];        // largest scaled score per token half and head (cold path)
__shared__ float mx_l[MX_HEADS];              // weight sums, exchanged once at the end
__shared__ unsigned mx_flag[2];               // "the weights beside me need a higher reference"

typedef short mx_s16x4 __attribute__((ext_vector_type(4)));
typedef short mx_s16x8 __attribute__((ext_vector_type(8)));
typedef __attribute__((address_space(3))) mx_s16x4 mx_lds_s16x4;

CL_DEVICE int mx_swz(int token) { return token & 6; }

// compile-time loop: f(MxI<B>{}), ..., f(MxI<E-1>{})
template <int I> struct MxI { static constexpr int value = I; };
template <int B, int E, class F>
CL_DEVICE void mx_for(F&& f) {
  if constexpr (B < E) {
    f(MxI<B>{});
    mx_for<B + 1, E>(f);
  }
}

// An iteration's matrix work in units of one A operand: a score unit (one 16-byte row read, two
// matrix ops: 32 features x both head tiles) or a value unit (one pair of transposing reads, four
// matrix ops: 16 features x four head tiles).  Order: groups of MX_SG score units, one value unit
// after each of the first groups, the other value units at the end (the softmax arithmetic of
// the finished scores runs beside those).
#ifndef CL_SG
#define CL_SG 6
#endif
#define MX_SG CL_SG
#define MX_NGROUPS ((MX_KJ + MX_SG - 1) / MX_SG)
#define MX_VEARLY (MX_NGROUPS < MX_FBW ? MX_NGROUPS : MX_FBW)
#define MX_UNITS (MX_KJ + MX_FBW)
#define MX_LAST_SCORE_UNIT (MX_KJ + MX_VEARLY - (MX_NGROUPS <= MX_FBW ? 1 : 0) - 1)
#ifndef CL_UNITS_AHEAD
#define CL_UNITS_AHEAD 6
#endif
#define MX_UNITS_AHEAD (CL_UNITS_AHEAD < MX_UNITS ? CL_UNITS_AHEAD : MX_UNITS)
#define MX_DMA_EVERY (MX_UNITS / MX_PANELS)    // a panel's load goes out every so many units
#ifndef CL_DMA_STAGGER
#define CL_DMA_STAGGER 0                      // (measured: staggering the waves' loads by unit is no faster)
#endif
#define MX_DMA_STAGGER (CL_DMA_STAGGER && MX_DMA_EVERY > 1)
#define MX_SOFTMAX_AT(k) (MX_LAST_SCORE_UNIT + 1 + (k) < MX_UNITS ? MX_LAST_SCORE_UNIT + 1 + (k) : MX_UNITS - 1)
constexpr bool mx_unit_is_value(int u) {
  int pos = 0;
  for (int grp = 0; grp < MX_NGROUPS; ++grp) {
    const int ns = MX_KJ - grp * MX_SG < MX_SG ? MX_KJ - grp * MX_SG : MX_SG;
    if (u < pos + ns) return false;
    pos += ns;
    if (grp < MX_VEARLY) {
      if (u == pos) return true;
      pos += 1;
    }
  }
  return true;
}
// 32-feature block of a score unit / 16-feature block (within the wave's features) of a value unit
constexpr int mx_unit_index(int u) {
  int pos = 0, scores = 0, values = 0;
  for (int grp = 0; grp < MX_NGROUPS; ++grp) {
    const int ns = MX_KJ - grp * MX_SG < MX_SG ? MX_KJ - grp * MX_SG : MX_SG;
    if (u < pos + ns) return scores + (u - pos);
    pos += ns;
    scores += ns;
    if (grp < MX_VEARLY) {
      if (u == pos) return values;
      pos += 1;
      values += 1;
    }
  }
  return values + (u - pos);
}
static_assert(!mx_unit_is_value(MX_LAST_SCORE_UNIT) && mx_unit_index(MX_LAST_SCORE_UNIT) == MX_KJ - 1, "unit order");
static_assert(mx_unit_is_value(MX_UNITS - 1) && mx_unit_index(MX_UNITS - 1) == MX_FBW - 1, "unit order");

// 16 bytes per lane, global -> LDS: the wave's 64 lanes fill 1 KiB starting at LDS byte address
// `lds_byte` + OFF (wave-uniform), lane l from `gptr` + OFF (the instruction's offset applies to
// both sides).  The compiler does not count this load: the kernel waits for it itself.
template <int OFF>
CL_DEVICE void mx_dma16(const void* gptr, unsigned lds_byte) {
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off offset:%2"
               :: "v"(gptr), "s"(__builtin_amdgcn_readfirstlane(lds_byte)), "n"(OFF) : "memory");
}

// wave w loads the 8-row group w of every panel: lane l takes row 8 w + l / 8 (a token of the
// step; CLAMP: tokens past the end are replaced by the last one) and the chunk that belongs in
// slot l % 8 of that row.  The same loader brings in the Q rows of 32 heads as an image.
template <int P, bool CLAMP>
CL_DEVICE void mx_issue_from(u32 lat_off, u32 pe_off, const elem_t* lat_rows, const elem_t* pe_rows, int t0,
                             unsigned stage_byte, int wave) {
  if constexpr (P < MX_PANELS) {
    constexpr int OFF = 128 * (P < MX_LAT_PANELS ? P : P - MX_LAT_PANELS);
    const unsigned lds_byte = stage_byte + (unsigned)(P * MX_PANEL * 2 + wave * 1024);
    if (CLAMP) {
      // tokens past the end are clamped onto the last one (their scores are masked later)
      const int lane = threadIdx.x & 63;
      const int r = 8 * wave + (lane >> 3);
      int t = t0 + r;
      t = t < CL_SKV - 1 ? t : CL_SKV - 1;
      const int chunk = (lane & 7) ^ mx_swz(r);
      const elem_t* src = P < MX_LAT_PANELS ? lat_rows + (i64)(t - t0) * CL_CKV + 64 * P + 8 * chunk
                                            : pe_rows + (i64)(t - t0) * CL_KPE + 64 * (P - MX_LAT_PANELS) + 8 * chunk;
      mx_dma16<0>(src, lds_byte);
    } else {
      const char* src = P < MX_LAT_PANELS ? reinterpret_cast<const char*>(lat_rows) + lat_off
                                          : reinterpret_cast<const char*>(pe_rows) + pe_off;
      mx_dma16<OFF>(src, lds_byte - OFF);
    }
    mx_issue_from<P + 1, CLAMP>(lat_off, pe_off, lat_rows, pe_rows, t0, stage_byte, wave);
  }
}

// one panel of the above (no clamping: whole steps only), for loads spread over an iteration
template <int P>
CL_DEVICE void mx_issue_panel(u32 lat_off, u32 pe_off, const elem_t* lat_rows, const elem_t* pe_rows,
                              unsigned stage_byte, int wave) {
  constexpr int OFF = 128 * (P < MX_LAT_PANELS ? P : P - MX_LAT_PANELS);
  const unsigned lds_byte = stage_byte + (unsigned)(P * MX_PANEL * 2 + wave * 1024);
  const char* src = P < MX_LAT_PANELS ? reinterpret_cast<const char*>(lat_rows) + lat_off
                                      : reinterpret_cast<const char*>(pe_rows) + pe_off;
  mx_dma16<OFF>(src, lds_byte - OFF);
}

#ifdef CL_DBG_TIMING
// debugging aid: wave 0 of every workgroup collects cycle-counter readings in LDS (no global
// stores that would disturb the load counter) and leaves them in its PL rows at the end
__shared__ unsigned mx_stamps[32];
#define MX_STAMP(k) if (threadIdx.x == 0) mx_stamps[k] = (unsigned)__builtin_readcyclecounter();
#define MX_STAMPS_OUT                                                                                 \
  __syncthreads();                                                                                    \
  if (threadIdx.x < 32)                                                                               \
    reinterpret_cast<unsigned*>(CL_ARG_PL)[(blockIdx.y * gridDim.x + blockIdx.x) * 32 + threadIdx.x] = mx_stamps[threadIdx.x];
#else
#define MX_STAMP(k)
#define MX_STAMPS_OUT
#endif

#if CL_EMIT_PARTIAL
extern "C" __global__ void __launch_bounds__(MX_THREADS, 1)
CL_PARTIAL_NAME(CL_PARTIAL_PARAMS) {
  MX_STAMP(0)
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int c = lane & 15, g = lane >> 4;
  const int th = wave & 1, hh = wave >> 1;     // score role: token half of a step, head half of the workgroup
  // Workgroups go to the eight XCDs (one L2 each) round-robin in launch order.  The head blocks
  // that read the same rows (one batch entry, one split) are given launch ids 8 apart, so they
  // run on one XCD at about the same time and all but the first find the rows in its L2.
  int b, split, hg_block;
  {
    constexpr int units = CL_BATCH * CL_SPLITS;            // (batch entry, split) pairs
    const int launch = blockIdx.y * gridDim.x + blockIdx.x;
    if (units % 8 == 0) {
      hg_block = (launch / 8) % MX_HEAD_GROUPS;
      const int unit = (launch % 8) + 8 * (launch / (8 * MX_HEAD_GROUPS));
      b = unit / CL_SPLITS;
      split = unit % CL_SPLITS;
    } else {
      split = blockIdx.y;
      b = blockIdx.x / MX_HEAD_GROUPS;
      hg_block = blockIdx.x % MX_HEAD_GROUPS;
    }
  }
  const elem_t* kv = CL_ARG_KV + (i64)b * CL_SKV * CL_CKV;
  const elem_t* kpe = CL_ARG_KPE + (i64)b * CL_SKV * CL_KPE;
  const i64 row0 = (i64)b * CL_HEADS + hg_block * MX_HEADS;   // flattened (batch, head) row of the workgroup's first head

  constexpr int n_steps = (CL_SKV + MX_STEP - 1) / MX_STEP;
  constexpr int per_split = (n_steps + CL_SPLITS - 1) / CL_SPLITS;
  const int step_begin = split * per_split;
  int step_end = step_begin + per_split;
  step_end = step_end < n_steps ? step_end : n_steps;
  const unsigned tiles_byte = (unsigned)(size_t)(__attribute__((address_space(3))) elem_t*)mx_tiles;

  f32x4 acc[4][MX_FBW];                // acc[ht][fb][r] = O[head 16 ht + c][feature 16 (FBW wave + fb) + 4 g + r]
  f32x4 l_acc = {0.f, 0.f, 0.f, 0.f};  // every component: weight sum of head 16 wave + c
#pragma unroll
  for (int ht = 0; ht < 4; ++ht)
#pragma unroll
    for (int fb = 0; fb < MX_FBW; ++fb) acc[ht][fb] = (f32x4){0.f, 0.f, 0.f, 0.f};
  float m_run[2] = {CL_NEG_BIG, CL_NEG_BIG};   // reference of head 32 hh + 16 ht + c (score role), uniform over g
  f32x4 st[2];                         // scores of the step whose weights were written last: st[ht][r] =
                                       // raw score (head 32 hh + 16 ht + c, token 16 th + 4 g + r of the step)

  if (step_begin < step_end) {
    // ---- set-up ---------------------------------------------------------------------------
    // Everything comes in through the global -> LDS path, so that the kernel's own load counter
    // sees every load and each wait is exact: the Q rows of the 64 heads first, as two images in
    // the layout of a step (rows = heads) parked in images 2 and 3, then steps 0 and 1.
    u32 lat_off, pe_off;               // byte offset of this lane's chunk from an image's first latent / rope row, panel 0
    {
      const int r = 8 * wave + (lane >> 3);
      const int chunk = (lane & 7) ^ mx_swz(r);
      lat_off = (u32)((r * CL_CKV + 8 * chunk) * 2);
      pe_off = (u32)((r * CL_KPE + 8 * chunk) * 2);
    }
#define MX_ISSUE(s)                                                                                   \
  {                                                                                                   \
    int s_ = (s) < step_end - 1 ? (s) : step_end - 1;   /* (the set-up may ask for one step too many) */ \
    const int t0_ = s_ * MX_STEP;                                                                     \
    mx_issue_from<0, MX_RAGGED>(lat_off, pe_off, kv + (i64)t0_ * CL_CKV, kpe + (i64)t0_ * CL_KPE, t0_, \
                                tiles_byte + (unsigned)((((s) - step_begin) % MX_STAGES) * MX_TILE * 2), wave); \
  }
#ifdef CL_DBG_NODMA
#define MX_DBG_ISSUE(s)
#else
#define MX_DBG_ISSUE(s) MX_ISSUE(s)
#endif
#define MX_WAITCNT(n) __builtin_amdgcn_s_waitcnt(0x0F70 | ((n) & 15) | (((n) >> 4) << 14))
#pragma unroll
    for (int half = 0; half < 2; ++half)
      mx_issue_from<0, false>(lat_off, pe_off, CL_ARG_Q + (row0 + 32 * half) * CL_CKV,
                              CL_ARG_QPE + (row0 + 32 * half) * CL_KPE, 0,
                              tiles_byte + (unsigned)((2 + half) * MX_TILE * 2), wave);
    MX_ISSUE(step_begin)
    if (threadIdx.x < MX_HEADS) mx_m[threadIdx.x] = CL_NEG_BIG;
    if (threadIdx.x < 2) mx_flag[threadIdx.x] = threadIdx.x == 0 ? 1u : 0u;   // the first step takes the cold path
    MX_STAMP(20)
    MX_WAITCNT(MX_UNITS_PER);          // the Q images have landed (this wave's share), step 0 may be in flight
    MX_STAMP(21)
    __syncthreads();
    // (a wave stalls at the issue of a load while the memory pipeline is full: what is not needed
    // first goes out later)
    MX_ISSUE(step_begin + 1)
    MX_STAMP(22)
    // Q fragments (B operand of the score product): lane (c, g) holds q[head 32 hh + 16 ht + c][32 j + 8 g .. +8].
    // They are only ever matrix-op operands: kept in the accumulation half of the register file,
    // which leaves the other half to the operands in flight.
    elem8 qf[2][MX_KJ];
    {
      const elem_t* qimg = mx_tiles + (2 + hh) * MX_TILE;
#pragma unroll
      for (int ht = 0; ht < 2; ++ht)
#pragma unroll
        for (int j = 0; j < MX_KJ; ++j) {
          const int q_lo = (16 * ht + c) * 64 + ((g ^ mx_swz(c)) << 3);
          qf[ht][j] = *reinterpret_cast<const elem8*>(qimg + (j >> 1) * MX_PANEL + (q_lo ^ ((4 * (j & 1)) << 3)));
        }
#pragma unroll
      for (int ht = 0; ht < 2; ++ht)
#pragma unroll
        for (int j = 0; j < MX_QA; ++j) asm volatile("" : "+a"(qf[ht][j]));
    }
    MX_STAMP(23)
    MX_WAITCNT(MX_UNITS_PER);          // step 0 has landed, step 1 may be in flight
    MX_STAMP(24)
    __syncthreads();                   // ... everybody's share; and everybody has taken its Q fragments: images 2, 3 are free
    MX_STAMP(25)
    if (step_begin + 2 < step_end) { MX_DBG_ISSUE(step_begin + 2) }

    elem8 ones;
#pragma unroll
    for (int i = 0; i < 8; ++i) ones[i] = to_elem(1.0f);

    // this lane's operand offsets inside an image (elements):
    //   score operand: token row 16 th + c, chunk g of a 32-feature block
    //   value operand: its 8-byte piece of the 4 (token) x 16 (feature) patch of lane group g
    const int a_lo = (16 * th + c) * 64 + ((g ^ mx_swz(c)) << 3);
    const int vtok = 4 * g + (c >> 2);
    const int v_lo = wave * (MX_FBW / 4) * MX_PANEL + vtok * 64 + (((((c & 3) >> 1)) ^ mx_swz(vtok)) << 3) + 4 * (c & 1);
    // weights: operand slot 8 G + 4 H + r of a head holds token 16 H + 4 G + r (the value operand's token order)
    const int p_read = c * MX_STEP + 8 * g;                    // + 16 ht * MX_STEP: B operand of head tile ht
    const int p_write = (32 * hh + c) * MX_STEP + 8 * g + 4 * th;   // + 16 ht * MX_STEP

    // scores of the 16 tokens x 32 heads of this wave from image `tile_s` (two accumulators per
    // head tile, even and odd 32-feature blocks: four independent chains in the matrix pipe)
#define MX_SCORE_MFMA(j)                                                                              \
    {                                                                                                 \
      const elem8 a_ = *reinterpret_cast<const elem8*>(tile_s + ((j) >> 1) * MX_PANEL +               \
                                                       (a_lo ^ ((4 * ((j) & 1)) << 3)));              \
      sa[0][(j) & 1] = mfma16(a_, qf[0][j], sa[0][(j) & 1]);                                          \
      sa[1][(j) & 1] = mfma16(a_, qf[1][j], sa[1][(j) & 1]);                                          \
    }
    // raw scores -> st (tokens past the end masked), then weights against the current reference
    // into weight buffer `buf`; a score more than MX_RESCALE_STEP above the reference raises the flag
#define MX_FINISH_SCORES(t0_step)                                                                     \
    _Pragma("unroll") for (int ht = 0; ht < 2; ++ht) {                                                \
      st[ht] = sa[ht][0] + sa[ht][1];                                                                 \
      if (MX_RAGGED) {                                                                                \
        _Pragma("unroll") for (int r = 0; r < 4; ++r)                                                 \
          if ((t0_step) + 16 * th + 4 * g + r >= CL_SKV) st[ht][r] = CL_NEG_BIG;                      \
      }                                                                                               \
    }
#define MX_WRITE_WEIGHTS_OF(buf, ht)                                                                  \
    {                                                                                                 \
      elem4 w_;                                                                                       \
      _Pragma("unroll") for (int r = 0; r < 4; ++r)                                                   \
        w_[r] = to_elem(fast_exp2(__builtin_fmaf(st[ht][r], CL_SCALE_LOG2E, -m_run[ht])));            \
      *reinterpret_cast<elem4*>(&mx_p[buf][0][0] + p_write + 16 * (ht) * MX_STEP) = w_;               \
    }
#define MX_WRITE_WEIGHTS(buf) MX_WRITE_WEIGHTS_OF(buf, 0) MX_WRITE_WEIGHTS_OF(buf, 1)

    {
      // scores of the first step (image 0); its weights are written by the cold path of the first iteration
      const elem_t* tile_s = mx_tiles;
      f32x4 sa[2][2];
#pragma unroll
      for (int ht = 0; ht < 2; ++ht) sa[ht][0] = sa[ht][1] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int j = 0; j < MX_KJ; ++j) MX_SCORE_MFMA(j)
      MX_FINISH_SCORES(step_begin * MX_STEP)
    }
    MX_STAMP(1)

    // The hot loop holds no rescaling code (with it inside, the compiler keeps copies of the
    // accumulators outside the matrix cores' registers on every step): a raised flag leaves the
    // loop, the cold block below handles it and the loop is entered again at the same step.
    // The front of that step then runs a second time: a second wait and barrier are harmless.
    int step = step_begin;
    for (;;) {
      bool flagged = false;
      while (step < step_end) {
        const int rel = step - step_begin;
        const int buf = rel & 1;
        // Image step+1: this wave's share has landed when at most one younger step's loads are
        // outstanding; the barrier makes that everybody's share, publishes the weights (and flag)
        // of `step`, and frees the image and the weight buffer of step-1 for reuse.
        if (step + 2 < step_end) {
          MX_WAITCNT(MX_UNITS_PER);
        } else {
          MX_WAITCNT(0);
        }
        __syncthreads();
        if (rel < 4) { MX_STAMP(2 + 4 * rel) }
        if (__builtin_amdgcn_readfirstlane(mx_flag[buf])) {
          flagged = true;
          break;
        }
        if (rel < 4) { MX_STAMP(4 + 4 * rel) }

        // ---- scores of step+1 beside the value product of step ---------------------------------
        // (after the split's last step the image of "step+1" is whatever its slot still holds:
        // those scores are computed like any others and never used)
        // The order below is the order of the instruction stream (a scheduling barrier closes
        // every unit): the operand read of unit u + MX_UNITS_AHEAD goes out before the matrix ops
        // of unit u, so that MX_UNITS_AHEAD reads are always in flight ahead of the matrix cores
        // (one wave per SIMD: nothing else hides the LDS latency).
        const elem_t* tile_v = mx_tiles + (rel % MX_STAGES) * MX_TILE;
        const elem_t* tile_s = mx_tiles + ((rel + 1) % MX_STAGES) * MX_TILE;
        const elem_t* pw = &mx_p[buf][0][0];
        elem8 pb[4];                     // weights of `step`: B operand per head tile
#pragma unroll
        for (int ht = 0; ht < 4; ++ht) pb[ht] = *reinterpret_cast<const elem8*>(pw + p_read + 16 * ht * MX_STEP);
        const elem8 pl = *reinterpret_cast<const elem8*>(pw + p_read + 16 * wave * MX_STEP);
        f32x4 sa[2][2];
#pragma unroll
        for (int ht = 0; ht < 2; ++ht) sa[ht][0] = sa[ht][1] = (f32x4){0.f, 0.f, 0.f, 0.f};
        // The loads of step + MX_AHEAD go out one panel at a time between the units: the path from
        // L2 into the compute unit moves 64 bytes per clock, and a wave that issues a load while
        // that path is busy stalls, matrix ops and all; four waves issuing a whole step at once
        // stand still for the 36 KiB transfer, spread out they hardly meet.  (Tokens past a ragged
        // end: the clamping loader, all panels in the first unit.)
        const int s_next = step + MX_AHEAD;
#ifdef CL_DBG_NODMA
        const bool issue_on = false;
#else
        const bool issue_on = s_next < step_end;
#endif
        const elem_t* next_lat = kv + (i64)s_next * MX_STEP * CL_CKV;
        const elem_t* next_pe = kpe + (i64)s_next * MX_STEP * CL_KPE;
        const unsigned next_byte = tiles_byte + (unsigned)(((rel + MX_AHEAD) % MX_STAGES) * MX_TILE * 2);
        const int dma_phase = wave % MX_DMA_EVERY;
        elem8 opnd[MX_UNITS];            // A operand of unit u (every index below is a compile-time constant)
        bool raise = false;
        auto issue = [&](auto U_) __attribute__((always_inline)) {
          constexpr int U = decltype(U_)::value;
          if constexpr (U < MX_UNITS) {
            constexpr int i = mx_unit_index(U);
            if constexpr (mx_unit_is_value(U)) {
              const elem_t* p_ = tile_v + (i >> 2) * MX_PANEL + (v_lo ^ (((2 * i) & 7) << 3));
              const mx_s16x4 lo_ = __builtin_amdgcn_ds_read_tr16_b64_v4i16((mx_lds_s16x4*)(p_));
              const mx_s16x4 hi_ = __builtin_amdgcn_ds_read_tr16_b64_v4i16((mx_lds_s16x4*)(p_ + 16 * 64));
              opnd[U] = __builtin_bit_cast(elem8, (mx_s16x8)__builtin_shufflevector(lo_, hi_, 0, 1, 2, 3, 4, 5, 6, 7));
            } else {
              opnd[U] = *reinterpret_cast<const elem8*>(tile_s + (i >> 1) * MX_PANEL + (a_lo ^ ((4 * (i & 1)) << 3)));
            }
          }
        };
        mx_for<0, MX_UNITS_AHEAD>(issue);
        mx_for<0, MX_UNITS>([&](auto U_) __attribute__((always_inline)) {
          constexpr int U = decltype(U_)::value;
          constexpr int i = mx_unit_index(U);
          issue(MxI<U + MX_UNITS_AHEAD>{});
          if constexpr (MX_RAGGED) {
            if constexpr (U == 0) {
              if (issue_on) { MX_ISSUE(s_next) }
            }
          } else if constexpr (MX_DMA_STAGGER) {
            // wave w takes the units u = MX_DMA_EVERY p + w % MX_DMA_EVERY: the waves run in step
            // (one barrier per iteration), so loads issued at the same unit would meet in the path
            if constexpr (U / MX_DMA_EVERY < MX_PANELS) {
              if (issue_on && U % MX_DMA_EVERY == dma_phase)
                mx_issue_panel<U / MX_DMA_EVERY>(lat_off, pe_off, next_lat, next_pe, next_byte, wave);
            }
          } else if constexpr (U % MX_DMA_EVERY == 0 && U / MX_DMA_EVERY < MX_PANELS) {
            if (issue_on) mx_issue_panel<U / MX_DMA_EVERY>(lat_off, pe_off, next_lat, next_pe, next_byte, wave);
          }
          if constexpr (U == 0) l_acc = mfma16(ones, pl, l_acc);
          if constexpr (mx_unit_is_value(U)) {
#pragma unroll
            for (int ht = 0; ht < 4; ++ht) acc[ht][i] = mfma16(opnd[U], pb[ht], acc[ht][i]);
          } else {
            sa[0][i & 1] = mfma16(opnd[U], qf[0][i], sa[0][i & 1]);
            sa[1][i & 1] = mfma16(opnd[U], qf[1][i], sa[1][i & 1]);
          }
          // the softmax arithmetic of step+1, in three pieces in the shadow of the value units
          // that follow the last score unit
          if constexpr (U == MX_SOFTMAX_AT(0)) {
            MX_FINISH_SCORES((step + 1) * MX_STEP)
#pragma unroll
            for (int ht = 0; ht < 2; ++ht) {
              const float v = fmaxf(fmaxf(st[ht][0], st[ht][1]), fmaxf(st[ht][2], st[ht][3])) * CL_SCALE_LOG2E;
              raise = raise | (v > m_run[ht] + MX_RESCALE_STEP);
            }
          }
          if constexpr (U == MX_SOFTMAX_AT(1)) MX_WRITE_WEIGHTS_OF(buf ^ 1, 0)
          if constexpr (U == MX_SOFTMAX_AT(2)) MX_WRITE_WEIGHTS_OF(buf ^ 1, 1)
          __builtin_amdgcn_sched_barrier(0);
        });
        if (__builtin_amdgcn_ballot_w64(raise) && lane == 0) mx_flag[buf ^ 1] = 1u;
        if (rel < 4) { MX_STAMP(5 + 4 * rel) }
        ++step;
      }
      if (!flagged) break;
      // ---- cold: raise the reference, rescale, redo the weights of `step` -----------------------
      const int buf = (step - step_begin) & 1;
#pragma unroll
      for (int ht = 0; ht < 2; ++ht) {
        float v = fmaxf(fmaxf(st[ht][0], st[ht][1]), fmaxf(st[ht][2], st[ht][3])) * CL_SCALE_LOG2E;
        v = fmaxf(v, lane_xor(v, lane, 16));
        v = fmaxf(v, lane_xor(v, lane, 32));
        if (g == 0) mx_cand[th][32 * hh + 16 * ht + c] = v;
      }
      __syncthreads();
      float alpha[4], m_new[4];
#pragma unroll
      for (int ht = 0; ht < 4; ++ht) {
        const int h = 16 * ht + c;
        const float m_old = mx_m[h];
        m_new[ht] = fmaxf(m_old, fmaxf(mx_cand[0][h], mx_cand[1][h]));
        alpha[ht] = fast_exp2(m_old - m_new[ht]);
      }
      if (step != step_begin) {          // (nothing has been accumulated before the first step)
#pragma unroll
        for (int ht = 0; ht < 4; ++ht)
#pragma unroll
          for (int fb = 0; fb < MX_FBW; ++fb) acc[ht][fb] *= alpha[ht];
      }
      // the wave-indexed picks below are selects, not register indexing
      l_acc *= wave == 0 ? alpha[0] : wave == 1 ? alpha[1] : wave == 2 ? alpha[2] : alpha[3];
      m_run[0] = hh ? m_new[2] : m_new[0];
      m_run[1] = hh ? m_new[3] : m_new[1];
      __syncthreads();                 // everybody has read the old references and the candidates
      if (th == 0 && g == 0) {
        mx_m[32 * hh + c] = m_run[0];
        mx_m[32 * hh + 16 + c] = m_run[1];
      }
      if (threadIdx.x == 0) mx_flag[buf] = 0u;
      MX_WRITE_WEIGHTS(buf)
      // (the barrier at the top of the loop publishes the weights and the cleared flag)
    }
    // no load may still be on its way into LDS when the workgroup ends
    MX_WAITCNT(0);
  }
  MX_STAMP(29)

  // ---- weight sums and references to every wave, then each wave writes its features of all heads
  if (g == 0) mx_l[16 * wave + c] = l_acc[0];
  if (step_begin >= step_end && threadIdx.x < MX_HEADS) mx_m[threadIdx.x] = CL_NEG_BIG;
  __syncthreads();
#pragma unroll
  for (int ht = 0; ht < 4; ++ht) {
    const int h = 16 * ht + c;
    const float l = mx_l[h];
    const float m = mx_m[h];
    const i64 orow = row0 + h;
    const int f0 = 16 * MX_FBW * wave + 4 * g;           // this lane's first feature of block 0
    const bool scalar_writer = wave == ht && g == 0;     // one lane per head writes the per-row scalars
#if CL_SPLITS > 1 && !CL_PO_ELEM
    const i64 prow = (i64)split * CL_TOTAL_ROWS + orow;
#pragma unroll
    for (int fb = 0; fb < MX_FBW; ++fb)
      *reinterpret_cast<f32x4*>(CL_ARG_PO + prow * CL_CKV + f0 + 16 * fb) = acc[ht][fb];
    if (scalar_writer) {
      CL_ARG_PM[prow] = m;
      CL_ARG_PL[prow] = l;
    }
#else
    const float inv = 1.0f / fmaxf(l, 1.0e-30f);
#if CL_SPLITS > 1
    const i64 prow = (i64)split * CL_TOTAL_ROWS + orow;
    elem_t* dst_row = CL_ARG_PO + prow * CL_CKV;
#ifndef CL_DBG_TIMING
    if (scalar_writer) {
      CL_ARG_PM[prow] = l > 0.f ? m + fast_log2(l) : CL_NEG_BIG;
      CL_ARG_PL[prow] = l > 0.f ? 1.0f : 0.f;
    }
#endif
#else
    elem_t* dst_row = CL_ARG_OUT + orow * CL_CKV;
#if CL_EMIT_LSE
    if (scalar_writer) CL_ARG_LSE[orow] = l > 0.f ? m + fast_log2(l) : CL_NEG_INF;
#endif
#endif
#pragma unroll
    for (int fb = 0; fb < MX_FBW; ++fb) {
      elem4 y;
#pragma unroll
      for (int r = 0; r < 4; ++r) y[r] = to_elem(acc[ht][fb][r] * inv);
      *reinterpret_cast<elem4*>(dst_row + f0 + 16 * fb) = y;
    }
#endif
  }
  MX_STAMP(30)
  MX_STAMPS_OUT
}
#endif  // CL_EMIT_PARTIAL
