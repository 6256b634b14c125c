// ---- split-KV decode attention (GQA / MQA / MHA), dense or paged KV --------------------------
//
// One workgroup owns one (kv-head unit, 16-row query tile, KV split).  Its waves walk the
// split's 32-token steps round-robin; nothing is staged through LDS on the way in: K and V
// rows go HBM -> registers as 16-byte loads and straight into the matrix cores.
//
//   scores^T (tokens x rows) = K (tokens x d) * Q^T        K rows are the A operand as loaded
//   out^T    (d x rows)     += V^T (d x tokens) * P^T      V is transposed 8x8 in registers;
//                                                          P^T is the score tile *in place*
//
// so every softmax quantity of query row c lives in lanes with lane%16 == c and the running
// max / sum / rescale never cross lanes except for one 4-way reduction per step.
// The softmax is exact and online: each wave carries (m, l, O) and waves, then splits, are
// merged by the usual max-rescale rule.  Emitter-supplied constants:
//   CL_HEAD_DIM  d (multiple of 32)      CL_VDIM     value width (multiple of 128, or 64)
//   CL_ROWS      query rows per kv unit  CL_WAVES    waves per workgroup
//   CL_SPLITS    KV splits               CL_PAGED    0 dense, 1 paged
//   CL_PAGE_SIZE tokens per page         CL_KV_HEADS kv heads in the cache (paged)
//   CL_Q_HEADS   query heads (paged)     CL_SKV      kv length (dense)
//   CL_SCALE_LOG2E softmax scale * log2(e) (dense; paged passes sm_scale at run time)
//   CL_EMIT_LSE  also write the base-2 log-sum-exp
//   CL_PREFETCH  steps of K/V in flight ahead of the one being computed (1 or 2)
//   CL_SKEW      0 = off.  The hardware deals workgroups out to the eight XCDs round-robin in launch
//                order, so with a grid whose x extent is a multiple of eight all splits of a unit
//                land on one XCD, and the XCDs do not stream equally fast (measured: the
//                odd-numbered ones about 5 % slower, whatever data they are given), so a kernel
//                dealt out in equal shares ends with its slowest XCD.  With CL_SKEW the units of
//                each group of eight are rotated by the split index, which spreads a unit's
//                splits over all XCDs, and of every pair of neighbouring splits the one on the
//                even XCD takes CL_SKEW thousandths of the pair's steps from the one on the odd
//                XCD.  Every step still belongs to exactly one split.  (Even split counts, grid x
//                a multiple of eight; the search times a few values.)
//   CL_CHUNK_PAGES  paged only, 0 = off.  1: work is cut into items of at most `chunk_pages`
//                pages (a run-time argument, 1..64, chosen by the host from the table length)
//                instead of a fixed number of splits per request, and a workgroup holds one wave
//                per kv head, so that the eight waves together stream whole contiguous token
//                rows of the cache and a long request costs many items rather than long ones.

#define ATT_RAISE_BY 8.0f
#ifndef CL_CHUNK_PAGES
#define CL_CHUNK_PAGES 0
#endif
#ifndef CL_SKEW
#define CL_SKEW 0
#endif
#ifndef CL_LOCKSTEP
#define CL_LOCKSTEP 0
#endif
#if CL_LOCKSTEP && !CL_CHUNK_PAGES
#error "waves in step: chunked items only (every wave walks the same steps)"
#endif
#if CL_LOCKSTEP
#define ATT_LOCKSTEP() __builtin_amdgcn_s_barrier();
#else
#define ATT_LOCKSTEP()
#endif
#if CL_SKEW && (CL_CHUNK_PAGES || CL_SPLITS % 2)
#error "skewed split ranges: an even number of splits, no chunked items"
#endif
#define ATT_STEP 32
#define ATT_KJ (CL_HEAD_DIM / 32)            // score MFMAs per 16 tokens
#define ATT_VC ((CL_VDIM + 127) / 128)       // 128-wide value chunks
#define ATT_ROW_TILES ((CL_ROWS + 15) / 16)

struct AttUnit {
  const elem_t* q;      // first query row of this tile (row stride CL_HEAD_DIM)
  const elem_t* k;      // dense: first K row of the unit; paged: cache base + head offset
  const elem_t* v;
  i64 k_stride, v_stride;   // elements between consecutive tokens of K and of V (their widths may differ)
  int kv_len;           // valid tokens
  int rows;             // real rows in this tile (1..16)
  const int* pages;     // paged: this request's slice of the page table
  int page_reg;         // chunked items: lane i holds the (clamped) id of the slice's page i
  int n_pages;          // paged: entries in that slice (>= 1 when kv_len > 0)
  int pool_pages;       // paged: pages in the cache; page ids are clamped below this
  i64 out_row;          // flattened (unit, row) index of the tile's first row
};

#if CL_PAGED && CL_CHUNK_PAGES
// An item's page ids were read once into one register per lane; a token's page id comes from
// the lane that holds it.  A page-table load per token would sit in the same in-order load
// queue as the K/V rows and make every prefetch wait for the rows of the step before it.
CL_DEVICE i64 att_token_row(const AttUnit& u, int t) {
  int pi = t / CL_PAGE_SIZE;
  pi = pi < u.n_pages ? pi : u.n_pages - 1;
  const i64 page = __builtin_amdgcn_ds_bpermute(pi << 2, u.page_reg);
  return page * CL_PAGE_SIZE + (t % CL_PAGE_SIZE);
}
#elif CL_PAGED
CL_DEVICE i64 att_token_row(const AttUnit& u, int t) {
  int pi = t / CL_PAGE_SIZE;
  pi = pi < u.n_pages ? pi : u.n_pages - 1;
  int pid = u.pages[pi];
  pid = pid < u.pool_pages - 1 ? pid : u.pool_pages - 1;
  pid = pid > 0 ? pid : 0;
  const i64 page = pid;
  return page * CL_PAGE_SIZE + (t % CL_PAGE_SIZE);
}
#else
CL_DEVICE i64 att_token_row(const AttUnit& u, int t) { (void)u; return (i64)t; }
#endif

struct AttTile {               // one 32-token step's K and V, as loaded
  u32x4 k[2][ATT_KJ];
  u32x4 v[ATT_VC][8];
};

// Issue the loads of the step starting at token t0.  Tokens past kv_len are clamped onto the
// last valid token (their scores are masked later), so no load leaves the tensor.
CL_DEVICE void att_load(const AttUnit& u, int t0, int c, int g, AttTile& tile) {
  const int last = u.kv_len - 1;
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    int t = t0 + 16 * h + c;
    t = t < last ? t : last;
    const elem_t* row = u.k + att_token_row(u, t) * u.k_stride + 8 * g;
#pragma unroll
    for (int j = 0; j < ATT_KJ; ++j) tile.k[h][j] = ld16(row + 32 * j);
  }
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    int t = t0 + (e < 4 ? 4 * g + e : 16 + 4 * g + (e - 4));
    t = t < last ? t : last;
    const elem_t* row = u.v + att_token_row(u, t) * u.v_stride;
#pragma unroll
    for (int vc = 0; vc < ATT_VC; ++vc) {
      int col = 128 * vc + 8 * c;
      if (CL_VDIM % 128 != 0) col = col < CL_VDIM - 8 ? col : CL_VDIM - 8;
      tile.v[vc][e] = ld16(row + col);
    }
  }
}

#if CL_CHUNK_PAGES
// Work items in page-table order: a new item starts at every multiple of chunk_pages table
// entries and at every request boundary, so item t = (chunk w) + (request b) for the one pair
// with chunk w overlapping request b.  Request b owns items b + p0/C .. b + (p1-1)/C.
static_assert(CL_PAGED && CL_ROWS <= 16 && CL_WAVES == CL_KV_HEADS, "chunked items: one wave per kv head");
CL_DEVICE int att_clamp_ptr(int p, int n_idx) { return p < 0 ? 0 : (p > n_idx ? n_idx : p); }
#endif

#if CL_EMIT_PARTIAL
// (one tile in flight and heads of up to 128: the kernel fits the 256 registers that let two waves
// share a SIMD, but the compiler only aims for that when told -- left alone it used 260 and halved the
// occupancy of the four-wave form; deeper rings and wider heads need more and are left alone)
// (the second figure of the launch bounds is waves per SIMD)
#if CL_PREFETCH == 1 && CL_HEAD_DIM <= 128 && CL_VDIM <= 128
#define ATT_WAVES_PER_SIMD 2
#else
#define ATT_WAVES_PER_SIMD 1
#endif
extern "C" __global__ void __launch_bounds__(CL_WAVES * 64, ATT_WAVES_PER_SIMD)
CL_PARTIAL_NAME(CL_PARTIAL_PARAMS) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int c = lane & 15, g = lane >> 4;
#if CL_CHUNK_PAGES
  const int split = 0, tile_id = 0;
  const int item = blockIdx.x;
#else
  const int split = blockIdx.y;
#if CL_SKEW
  // this workgroup runs on XCD blockIdx.x % 8 (grid x is a multiple of eight); the unit tile it
  // works for is rotated within its group of eight by the split index
  const int xcd = blockIdx.x & 7;
  const int unit_tile = (blockIdx.x & ~7) | ((xcd + split) & 7);
#else
  const int unit_tile = blockIdx.x;
#endif
  const int tile_id = unit_tile % ATT_ROW_TILES;
  const int unit = unit_tile / ATT_ROW_TILES;
#endif

  AttUnit u;
  u.rows = CL_ROWS - 16 * tile_id < 16 ? CL_ROWS - 16 * tile_id : 16;
#if CL_CHUNK_PAGES
  // the request whose items include `item`: the last b with b + indptr[b] / C <= item
  const ClRequest found = cl_find_request(CL_ARG_INDPTR, batch, n_idx, chunk_pages, 1, item, lane);
  const int req = found.req, p0 = found.p0, p1 = found.p1;
  const int head = wave;
  const int chunk = item - req;
  const int lo = p0 > chunk * chunk_pages ? p0 : chunk * chunk_pages;
  const int hi = p1 < (chunk + 1) * chunk_pages ? p1 : (chunk + 1) * chunk_pages;
  if (hi <= lo) return;                               // an index no (chunk, request) pair maps to
  {
    int lastp = CL_PAGE_SIZE;
#if CL_PAGE_SIZE > 1
    if (hi == p1) {
      lastp = CL_ARG_LAST[req];
      lastp = lastp > 0 ? (lastp < CL_PAGE_SIZE ? lastp : CL_PAGE_SIZE) : 0;
    }
#endif
    u.kv_len = (hi - lo - 1) * CL_PAGE_SIZE + lastp;
  }
  u.pages = CL_ARG_INDICES + lo;
  u.n_pages = hi - lo;
  u.pool_pages = num_pages;
  {
    int pid = u.pages[lane < u.n_pages ? lane : u.n_pages - 1];
    pid = pid < num_pages - 1 ? pid : num_pages - 1;
    u.page_reg = pid > 0 ? pid : 0;
  }
  u.k_stride = (i64)CL_KV_HEADS * CL_HEAD_DIM;
  u.v_stride = (i64)CL_KV_HEADS * CL_VDIM;
  u.k = CL_ARG_K + (i64)head * CL_HEAD_DIM;
  u.v = CL_ARG_V + (i64)head * CL_VDIM;
  u.out_row = (i64)req * CL_Q_HEADS + (i64)head * CL_ROWS;
  u.q = CL_ARG_Q + u.out_row * CL_HEAD_DIM;
  const float scale2 = sm_scale * 1.4426950408889634f;
#elif CL_PAGED
  // unit = request * kv_heads + kv head.  The request's length follows the page-granular
  // CSR: every page but the last is full, the last holds kv_last_page_len tokens, and the
  // sum is clamped to the pages the request owns.
  const int req = unit / CL_KV_HEADS, head = unit % CL_KV_HEADS;
  const int p0 = CL_ARG_INDPTR[req], p1 = CL_ARG_INDPTR[req + 1];
  int n_pages = p1 - p0;
  n_pages = n_pages > 0 ? n_pages : 0;
  {
    int avail = n_idx - p0;                       // never index past the table itself
    n_pages = n_pages < avail ? n_pages : (avail > 0 ? avail : 0);
  }
#if CL_PAGE_SIZE > 1
  int lastp = CL_ARG_LAST[req];
  lastp = lastp > 0 ? lastp : 0;
  int full = n_pages - 1 > 0 ? n_pages - 1 : 0;
  int kv_len = full * CL_PAGE_SIZE + lastp;
  kv_len = kv_len < n_pages * CL_PAGE_SIZE ? kv_len : n_pages * CL_PAGE_SIZE;
#else
  int kv_len = n_pages;
#endif
  u.kv_len = kv_len;
  u.pages = CL_ARG_INDICES + p0;
  u.page_reg = 0;
  u.n_pages = n_pages;
  u.pool_pages = num_pages;
  u.k_stride = (i64)CL_KV_HEADS * CL_HEAD_DIM;
  u.v_stride = (i64)CL_KV_HEADS * CL_VDIM;
  u.k = CL_ARG_K + (i64)head * CL_HEAD_DIM;
  u.v = CL_ARG_V + (i64)head * CL_VDIM;
  u.out_row = ((i64)req * CL_Q_HEADS + (i64)head * CL_ROWS) + 16 * tile_id;
  u.q = CL_ARG_Q + u.out_row * CL_HEAD_DIM;
  const float scale2 = sm_scale * 1.4426950408889634f;
#else
  u.kv_len = CL_SKV;
  u.page_reg = 0;
  u.pages = nullptr;
  u.n_pages = 0;
  u.pool_pages = 0;
  u.k_stride = CL_HEAD_DIM;
  u.v_stride = CL_VDIM;
  u.k = CL_ARG_K + (i64)unit * CL_SKV * CL_HEAD_DIM;
  u.v = CL_ARG_V + (i64)unit * CL_SKV * CL_VDIM;
  u.out_row = (i64)unit * CL_ROWS + 16 * tile_id;
  u.q = CL_ARG_Q + u.out_row * CL_HEAD_DIM;
  const float scale2 = CL_SCALE_LOG2E;
#endif

  // This split's steps: ceil(n_steps / SPLITS) each; a trailing split may own none.
  const int n_steps = (u.kv_len + ATT_STEP - 1) / ATT_STEP;
#if CL_CHUNK_PAGES
  const int step_begin = 0, step_end = n_steps;      // the item is the unit of work: no further cut
  (void)split;
#elif CL_SKEW
  // splits 2k and 2k + 1 share ceil(n_steps / (SPLITS / 2)) steps; the one on the even XCD takes
  // the larger share.  XCD parity = parity of (unit tile - split): exactly one of a pair is even.
  int step_begin, step_end;
  {
    const int per_pair = (n_steps + CL_SPLITS / 2 - 1) / (CL_SPLITS / 2);
    int lo = (split >> 1) * per_pair, hi = lo + per_pair;
    lo = lo < n_steps ? lo : n_steps;
    hi = hi < n_steps ? hi : n_steps;
    const int len = hi - lo;
    int big = (len + 1) / 2 + ((len / 2) * CL_SKEW + 500) / 1000;
    big = big < len ? big : len;
    const bool even_xcd = (xcd & 1) == 0;
    const int first = (split & 1) == 0 ? (even_xcd ? big : len - big) : (even_xcd ? len - big : big);
    step_begin = (split & 1) == 0 ? lo : lo + first;
    step_end = (split & 1) == 0 ? lo + first : hi;
  }
#else
  const int per_split = (n_steps + CL_SPLITS - 1) / CL_SPLITS;
  const int step_begin = split * per_split;
  int step_end = step_begin + per_split;
  step_end = step_end < n_steps ? step_end : n_steps;
#endif

  // Query rows as the B operand: lane (c, g) holds Q[row c][32 j + 8 g .. +8]; padded rows are 0.
  elem8 qf[ATT_KJ];
  {
    const bool live = c < u.rows;
    const elem_t* row = u.q + (i64)(live ? c : 0) * CL_HEAD_DIM + 8 * g;
#pragma unroll
    for (int j = 0; j < ATT_KJ; ++j) {
      u32x4 raw = ld16(row + 32 * j);
      if (!live) raw = (u32x4){0u, 0u, 0u, 0u};
      qf[j] = as_elem8(raw);
    }
  }

  float m_run = CL_NEG_BIG;   // reference point of the row's scaled scores (log2 domain, within 8 of their running max), uniform over g
  float l_run = 0.f;          // this lane's share of the running sum
  f32x4 acc[ATT_VC][8];       // acc[vc][j][r] = O[row c][128 vc + 32 g + 8 r + j]
#pragma unroll
  for (int vc = 0; vc < ATT_VC; ++vc)
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[vc][j] = (f32x4){0.f, 0.f, 0.f, 0.f};

  // Ring of CL_PREFETCH + 1 register tiles: while step n is in the matrix cores the loads of
  // steps n+1 .. n+CL_PREFETCH are in flight.  The ring position is a compile-time constant of
  // the unrolled inner loop, so every tile stays in registers.
  AttTile ring[CL_PREFETCH + 1];
#if CL_CHUNK_PAGES
#define ATT_WSTRIDE 1                 // every wave walks all steps of the item for its own head
  const int step0 = step_begin;
#else
#define ATT_WSTRIDE CL_WAVES
  const int step0 = step_begin + wave;
#endif
  // Inside the loop prefetch loads are issued unconditionally (a branch around them would make the
  // hardware load counter differ between paths, and the waits the compiler then has to insert drain
  // the prefetch before every value product): the loop runs only while the step CL_PREFETCH ahead of
  // each of its steps exists, and the last steps follow as straight-line code that asks for nothing
  // past the wave's last step.
// One 32-token step: asks for the step CL_PREFETCH ahead into the ring slot the previous step left, then
// multiplies the slot R: scores^T for the two 16-token halves, weights, value product.
// The softmax reference point of a row is raised only when a score passes it by more than 8 (a factor
// 2^8: weights stay below 256, softmax does not depend on the reference point), so after the first steps
// of a split the maxima are not even compared across the four lane groups and the accumulators are not
// rescaled: both happen only when some lane asks (the two ballots are wave-uniform and cold).  Masked
// slots hold CL_NEG_BIG; while a whole row is still masked its reference equals it too, so the weights
// test the mask itself rather than trusting exp2 of a zero difference.  The row sum adds up the weights
// before they are rounded to the element type (as the reference's kernels do): it normalises the output
// and is the lse, which at bf16 showed the rounding (1 - 2e-3) for requests of a few tokens otherwise.
// CL_LOCKSTEP (chunked items): the waves of a workgroup, one per kv head, meet at a barrier before every
// step.  Left alone they drift apart (the older wave of a SIMD is served first: in a 1024-token item the
// first wave is done after 88 us, the last after 155) and the item is as slow as its slowest wave; in step,
// the eight 256-byte pieces of a token row are also asked for together.  Every wave of an item walks the same
// steps, so every wave reaches every barrier.
// (A macro, so that the loop below holds no branch out of its body: with one, the compiler must assume
// at the loop head that loads of the skipped part are still on their way into registers it is about to
// reuse for addresses, and it waits for the current tile before it asks for the next.)
#define ATT_ONE_STEP(R, STEP, LOAD)                                                                 \
    {                                                                                               \
      ATT_LOCKSTEP()                                                                                \
      if (LOAD) att_load(u, ((STEP) + CL_PREFETCH * ATT_WSTRIDE) * ATT_STEP, c, g, ring[((R) + CL_PREFETCH) % (CL_PREFETCH + 1)]); \
      const AttTile& cur = ring[R];                                                                 \
      const int t0 = (STEP) * ATT_STEP;                                                             \
                                                                                                    \
      float s[8];                                                                                   \
_Pragma("unroll")                                                                                   \
      for (int h = 0; h < 2; ++h) {                                                                 \
        f32x4 st = (f32x4){0.f, 0.f, 0.f, 0.f};                                                     \
_Pragma("unroll")                                                                                   \
        for (int j = 0; j < ATT_KJ; ++j) st = mfma16(as_elem8(cur.k[h][j]), qf[j], st);             \
_Pragma("unroll")                                                                                   \
        for (int q = 0; q < 4; ++q) {                                                               \
          const int t = t0 + 16 * h + 4 * g + q;                                                    \
          s[4 * h + q] = t < u.kv_len ? st[q] * scale2 : CL_NEG_BIG;                                \
        }                                                                                           \
      }                                                                                             \
      float mx = s[0];                                                                              \
_Pragma("unroll")                                                                                   \
      for (int i = 1; i < 8; ++i) mx = fmaxf(mx, s[i]);                                             \
      float alpha = 1.0f;                                                                           \
      if (__builtin_amdgcn_ballot_w64(mx > m_run + ATT_RAISE_BY)) {                                 \
        mx = fmaxf(mx, lane_xor(mx, lane, 16));                                                     \
        mx = fmaxf(mx, lane_xor(mx, lane, 32));                                                     \
        if (mx > m_run + ATT_RAISE_BY) {                                                            \
          alpha = fast_exp2(m_run - mx);                                                            \
          m_run = mx;                                                                               \
        }                                                                                           \
      }                                                                                             \
      const float m_new = m_run;                                                                    \
      elem8 pf;                                                                                     \
      float psum = 0.f;                                                                             \
_Pragma("unroll")                                                                                   \
      for (int i = 0; i < 8; ++i) {                                                                 \
        float p = s[i] > 0.5f * CL_NEG_BIG ? fast_exp2(s[i] - m_new) : 0.f;                         \
        psum += p;                                                                                  \
        pf[i] = to_elem(p);                                                                         \
      }                                                                                             \
      l_run = l_run * alpha + psum;                                                                 \
                                                                                                    \
      if (__builtin_amdgcn_ballot_w64(alpha != 1.0f)) {                                             \
_Pragma("unroll")                                                                                   \
        for (int vc = 0; vc < ATT_VC; ++vc)                                                         \
_Pragma("unroll")                                                                                   \
          for (int j = 0; j < 8; ++j) acc[vc][j] *= alpha;                                          \
      }                                                                                             \
_Pragma("unroll")                                                                                   \
      for (int vc = 0; vc < ATT_VC; ++vc) {                                                         \
        u32x4 vt[8];                                                                                \
        transpose8x8(cur.v[vc], vt);                                                                \
_Pragma("unroll")                                                                                   \
        for (int j = 0; j < 8; ++j) acc[vc][j] = mfma16(as_elem8(vt[j]), pf, acc[vc][j]);           \
      }                                                                                             \
    }
  // A wave with steps of its own (one branch around prologue and loop together, so that the wait for
  // the Q fragments sits behind the first tiles' loads, not at a join that knows nothing of them).
  if (step0 < step_end) {
#pragma unroll
    for (int i = 0; i < CL_PREFETCH; ++i)
      if (step0 + i * ATT_WSTRIDE < step_end) att_load(u, (step0 + i * ATT_WSTRIDE) * ATT_STEP, c, g, ring[i]);
    int base = step0;
    for (; base + 2 * CL_PREFETCH * ATT_WSTRIDE < step_end; base += (CL_PREFETCH + 1) * ATT_WSTRIDE) {
#pragma unroll
      for (int r = 0; r <= CL_PREFETCH; ++r) ATT_ONE_STEP(r, base + r * ATT_WSTRIDE, true)
    }
    // (at most 2 * CL_PREFETCH steps are left)
#pragma unroll
    for (int r = 0; r < 2 * CL_PREFETCH; ++r)
      if (base + r * ATT_WSTRIDE < step_end)
        ATT_ONE_STEP(r % (CL_PREFETCH + 1), base + r * ATT_WSTRIDE, base + (r + CL_PREFETCH) * ATT_WSTRIDE < step_end)
  }

  l_run += lane_xor(l_run, lane, 16);
  l_run += lane_xor(l_run, lane, 32);
#if CL_WAVES > 1 && !CL_CHUNK_PAGES
  // ---- the workgroup's waves merged into its first one through LDS: every other wave leaves its
  // reference points, weight sums and accumulators as they lie in its registers (one 16-byte piece
  // per lane and accumulator: whole 1 KiB rows), and the first wave folds them into its own by the
  // max-rescale rule: one LDS round trip for all of them --------------------------------------
  {
    extern __shared__ float att_lds[];
    f32x4* sh_o = reinterpret_cast<f32x4*>(att_lds);                          // [WAVES - 1][8 ATT_VC][64]
    float* sh_m = att_lds + (CL_WAVES - 1) * 8 * ATT_VC * 64 * 4;              // [WAVES - 1][16]
    float* sh_l = sh_m + (CL_WAVES - 1) * 16;                                  // [WAVES - 1][16]
    if (wave > 0) {
#pragma unroll
      for (int vc = 0; vc < ATT_VC; ++vc)
#pragma unroll
        for (int j = 0; j < 8; ++j) sh_o[((wave - 1) * 8 * ATT_VC + 8 * vc + j) * 64 + lane] = acc[vc][j];
      if (g == 0) {
        sh_m[(wave - 1) * 16 + c] = m_run;
        sh_l[(wave - 1) * 16 + c] = l_run;
      }
    }
    __syncthreads();
    if (wave > 0) return;
    float ms[CL_WAVES - 1], m = m_run;
#pragma unroll
    for (int w = 0; w < CL_WAVES - 1; ++w) {
      ms[w] = sh_m[w * 16 + c];
      m = fmaxf(m, ms[w]);
    }
    // (a wave without steps holds m = -huge, l = 0, zeros: factor 1 of nothing when every wave is empty)
    const float f0 = fast_exp2(m_run - m);
    l_run *= f0;
#pragma unroll
    for (int vc = 0; vc < ATT_VC; ++vc)
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[vc][j] *= f0;
#pragma unroll
    for (int w = 0; w < CL_WAVES - 1; ++w) {
      const float f = fast_exp2(ms[w] - m);
      l_run += sh_l[w * 16 + c] * f;
#pragma unroll
      for (int vc = 0; vc < ATT_VC; ++vc)
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[vc][j] += sh_o[(w * 8 * ATT_VC + 8 * vc + j) * 64 + lane] * f;
    }
    m_run = m;
  }
#endif
  // ---- the rows leave straight from the accumulators of the wave that owns them (the first wave of
  // a workgroup; every wave of a chunked item, which owns one kv head): lane (c, g) holds, of row c,
  // the eight neighbours from 128 vc + 32 g + 8 r on for every r --------------------------------
  if (c < u.rows) {
    const i64 orow = u.out_row + c;
#if CL_CHUNK_PAGES
    const i64 prow = (i64)item * CL_Q_HEADS + (i64)head * CL_ROWS + c;      // partials are (item, query head[, d])
    float* dst = CL_ARG_PO + prow * CL_VDIM;
    (void)orow;
#elif CL_SPLITS > 1
    const i64 prow = (i64)split * CL_TOTAL_ROWS + orow;
    float* dst = CL_ARG_PO + prow * CL_VDIM;
#else
    elem_t* dst = CL_ARG_OUT + orow * CL_VDIM;
    const float inv_l = 1.0f / fmaxf(l_run, 1.0e-30f);     // an empty request has l == 0: 0 / floor = 0
#endif
#pragma unroll
    for (int vc = 0; vc < ATT_VC; ++vc)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int d0 = 128 * vc + 32 * g + 8 * r;
        if (CL_VDIM % 128 != 0 && d0 >= CL_VDIM) continue;
#if CL_SPLITS > 1 || CL_CHUNK_PAGES
        *reinterpret_cast<f32x4*>(dst + d0) = (f32x4){acc[vc][0][r], acc[vc][1][r], acc[vc][2][r], acc[vc][3][r]};
        *reinterpret_cast<f32x4*>(dst + d0 + 4) = (f32x4){acc[vc][4][r], acc[vc][5][r], acc[vc][6][r], acc[vc][7][r]};
#else
        elem8 y;
#pragma unroll
        for (int j = 0; j < 8; ++j) y[j] = to_elem(acc[vc][j][r] * inv_l);
        *reinterpret_cast<elem8*>(dst + d0) = y;
#endif
      }
    if (g == 0) {
#if CL_SPLITS > 1 || CL_CHUNK_PAGES
      CL_ARG_PM[prow] = m_run;
      CL_ARG_PL[prow] = l_run;
#elif CL_EMIT_LSE
      CL_ARG_LSE[orow] = l_run > 0.f ? m_run + fast_log2(l_run) : CL_NEG_INF;
#endif
    }
  }

}
#endif  // CL_EMIT_PARTIAL

