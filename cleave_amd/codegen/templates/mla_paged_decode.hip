// ---- paged MLA decode: per request, out = softmax((q kv^T + q_pe k_pe^T) * sm_scale) kv with the
// latent (kv) and rope (k_pe) rows gathered through a token table (page size 1) ----------------
//
// One wave per work item and 16-head group.  An item is a request (single kernel) or, with
// CL_CHUNKED, a slice of at most `chunk_pages` table entries of one request (a new item starts
// at every multiple of chunk_pages entries and at every request boundary, as in the chunked GQA
// decode; the combine folds a request's items).  The wave walks its tokens in steps of 32: the
// latent and rope rows of a step go from global memory straight into LDS (16 bytes per lane, the
// row of every lane looked up in the table) as the token-major image of the dense MLA kernel:
//   tile  [D/64][32][64]   64-feature panels, 128-byte token rows, 16-byte chunk ^ (token & 6)
// CL_MP_STAGES images (2, 3 or 4), the rows of the next CL_MP_STAGES - 1 steps in flight while the
// matrix cores work on the current one: a step's rows take about a microsecond to arrive from the
// cache, twice a step's matrix work, so with two images a lone item advances one round trip per
// step (nothing else runs on its compute unit to fill the wait), with three or four its steps
// cost what their matrix work costs; many resident items hide the same wait by their number, and
// two images let a compute unit hold two of them.
// Table entries are read 256 at a time into four registers per lane (entry 64 k + lane in
// register k) one window ahead; a lane fetches the entry of the row it loads with a cross-lane
// read.  Scores, softmax and value product are the dense kernel's (16 heads per wave, Q fragments
// resident, fixed softmax reference raised outside the hot loop).
//
// CL_PREFILL: causal prefill over ragged query rows -- an item is up to CL_MP_TOK consecutive query
// tokens of one request (a new item at every multiple of CL_MP_TOK packed tokens and at every
// request boundary), one wave per token (rows = its 16 heads), and the keys the item's last token
// may see: the waves of an item share the two images (each loads a share of a step's rows, one
// barrier per step) and every wave masks by its own token's causal limit; out and lse are per
// query token.  Four tokens per item quarter the traffic into the CU and put eight waves on a CU
// where single-token items have two (an item's images take 72 KB of LDS whatever its wave count).
//
// CL_MP_KSPLIT = 2 (single kernel; prefill: one token per item): two waves share an item's keys
// instead -- wave w walks steps w, w + 2, .. through images of its own, with no barrier between
// them, and at the end the second leaves its reference point, sums and accumulators in LDS for
// the first to fold into its own by the max-rescale rule.  A lone wave issues an instruction
// every four or five clocks and a step is about 600 of them, so an item alone on its compute unit
// takes 1.4 us per 32 keys whatever is in flight: two waves halve that where there are too few
// items to fill the chip.
//
//   CL_HEADS (multiple of 16)  CL_CKV  CL_KPE (multiples of 64)  CL_CHUNKED  CL_PREFILL
//   run-time: batch, num_pages, n_idx [, chunk_pages]; scalar sm_scale (> 0 or not: the
//   maximum is taken over scaled scores)

#ifndef CL_PREFILL
#define CL_PREFILL 0
#endif
#ifndef CL_MP_TOK
#define CL_MP_TOK 1
#endif
#ifndef CL_MP_KSPLIT
#define CL_MP_KSPLIT 1
#endif
#define MP_KS CL_MP_KSPLIT                                            // waves that deal an item's steps out between them
#define MP_TOKENS (CL_PREFILL && MP_KS == 1 ? CL_MP_TOK : 1)          // query tokens per work item
#define MP_WAVES (MP_KS > 1 ? MP_KS : MP_TOKENS)                      // waves per workgroup
#define MP_SHARE (MP_KS > 1 ? 1 : MP_WAVES)                           // waves that load and read one image together
static_assert(MP_TOKENS == 1 || MP_TOKENS == 2 || MP_TOKENS == 4, "1, 2 or 4 tokens per prefill item");
static_assert(MP_KS == 1 || (MP_KS == 2 && !CL_CHUNKED && (!CL_PREFILL || CL_MP_TOK == 1)),
              "keys shared between two waves: single kernel, one token per item");
#define MP_STEP 32
#define MP_D (CL_CKV + CL_KPE)
#define MP_PANEL (MP_STEP * 64)
#define MP_PANELS (MP_D / 64)
#define MP_LAT_PANELS (CL_CKV / 64)
#define MP_TILE (MP_PANELS * MP_PANEL)
#define MP_KJ (MP_D / 32)
#define MP_FB (CL_CKV / 16)
#define MP_WINDOW 256                          // table entries held in registers at a time
#ifndef CL_MP_STAGES
#define CL_MP_STAGES 2
#endif
#define MP_AHEAD (CL_MP_STAGES - 1)            // steps whose rows are asked for ahead of the one in the matrix cores
#define MP_UNITS ((4 / MP_SHARE) * MP_PANELS)  // loads one wave issues for a step
static_assert(CL_MP_STAGES >= 2 && CL_MP_STAGES <= 4, "two to four images");
static_assert((MP_AHEAD - 1) * MP_UNITS <= 63, "the load counter holds the loads of the steps in flight behind the awaited one");
#define MP_RESCALE_STEP 8.0f
#ifndef CL_LDS_AHEAD
#define CL_LDS_AHEAD 8
#endif
static_assert(CL_CKV % 64 == 0 && CL_KPE % 64 == 0, "latent and rope widths are whole 64-feature panels");
static_assert(CL_HEADS % 16 == 0, "16 heads per wave");

__shared__ __attribute__((aligned(1024))) elem_t mp_tiles[MP_KS * CL_MP_STAGES * MP_TILE];   // (a key-sharing wave has images of its own)
static_assert(MP_KS == 1 || (MP_FB * 64 * 4 + 3 * 64) * 4 <= MP_TILE * 2, "a wave's sums fit one of its images");

typedef short mp_s16x4 __attribute__((ext_vector_type(4)));
typedef short mp_s16x8 __attribute__((ext_vector_type(8)));
typedef __attribute__((address_space(3))) mp_s16x4 mp_lds_s16x4;

CL_DEVICE int mp_swz(int token) { return token & 6; }
CL_DEVICE int mp_clamp(int v, int lo, int hi) { return v < lo ? lo : (v > hi ? hi : v); }

#define MP_WAITCNT(n) __builtin_amdgcn_s_waitcnt(0x0F70 | ((n) & 15) | (((n) >> 4) << 14))
// rows (16 lanes) 1 and 3 of `a` trade places with rows 0 and 2 of `b`
CL_DEVICE void mp_swap_rows16(unsigned& a, unsigned& b) {
  asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 0" : "+v"(a), "+v"(b));
}

// 16 bytes per lane, global -> LDS: the wave's 64 lanes fill 1 KiB starting at LDS byte address
// `lds_byte` + OFF (wave-uniform), lane l from `gptr` + OFF.  Not counted by the compiler: the
// kernel waits for it itself.
template <int OFF>
CL_DEVICE void mp_dma16(const void* gptr, unsigned lds_byte) {
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off offset:%2"
               :: "v"(gptr), "s"(__builtin_amdgcn_readfirstlane(lds_byte)), "n"(OFF) : "memory", "m0");
}

// panels P.. of row group RG (token rows 8 RG + lane / 8 of the step) from this lane's row
template <int P>
CL_DEVICE void mp_issue_row_group(const char* lat_src, const char* pe_src, unsigned group_byte) {
  if constexpr (P < MP_PANELS) {
    constexpr int OFF = 128 * (P < MP_LAT_PANELS ? P : P - MP_LAT_PANELS);
    mp_dma16<OFF>(P < MP_LAT_PANELS ? lat_src : pe_src, group_byte + (unsigned)(P * MP_PANEL * 2) - OFF);
    mp_issue_row_group<P + 1>(lat_src, pe_src, group_byte);
  }
}

#if CL_EMIT_PARTIAL
extern "C" __global__ void __launch_bounds__(64 * MP_WAVES)
CL_PARTIAL_NAME(CL_PARTIAL_PARAMS) {
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int c = lane & 15, g = lane >> 4;
  const int head0 = 16 * blockIdx.y;
  const int tw = MP_KS > 1 ? 0 : wave;                // which of the item's tokens (or load shares) is this wave's
  const int kw = MP_KS > 1 ? wave : 0;                // which of the item's steps: kw, kw + MP_KS, ..
#if CL_CHUNKED
  const int item = blockIdx.x;
  // the request whose items include `item`: the last b with b + indptr[b] / C <= item
  const ClRequest found = cl_find_request(CL_ARG_INDPTR, batch, n_idx, chunk_pages, 1, item, lane);
  const int req = found.req, p0 = found.p0, p1 = found.p1;
  const int chunk = item - req;
  const int lo = p0 > chunk * chunk_pages ? p0 : chunk * chunk_pages;
  const int hi = p1 < (chunk + 1) * chunk_pages ? p1 : (chunk + 1) * chunk_pages;
  if (hi <= lo) return;                               // an index no (chunk, request) pair maps to
#elif CL_PREFILL
  // causal prefill: the request whose items include `item` is the last b with
  // b + qo_indptr[b] / MP_TOKENS <= item; token t of it sees the keys kv_pos <= kv_len - q_len + (t - q0)
  const int item = blockIdx.x;
  const ClRequest found = cl_find_request(CL_ARG_QINDPTR, batch, total_q, MP_TOKENS, 1, item, lane, CL_ARG_INDPTR, n_idx);
  const int req = found.req, q0 = found.p0, q1 = found.p1;
  const int chunk = item - req;
  const int t_lo = q0 > chunk * MP_TOKENS ? q0 : chunk * MP_TOKENS;
  const int t_hi = q1 < (chunk + 1) * MP_TOKENS ? q1 : (chunk + 1) * MP_TOKENS;
  if (t_hi <= t_lo) return;                           // an index no (chunk, request) pair maps to
  const bool tok_live = t_lo + tw < t_hi;             // this wave's token (a wave past the item's tokens only helps load)
  const int qtok = tok_live ? t_lo + tw : t_lo;
  const int lo = found.s0;
  int hi, n_tok_own;
  {
    int kv_len = found.s1 - lo;
    kv_len = kv_len > 0 ? kv_len : 0;
    const int ext_own = kv_len - (q1 - q0) + (qtok - q0) + 1, ext_all = kv_len - (q1 - q0) + (t_hi - 1 - q0) + 1;
    n_tok_own = tok_live ? mp_clamp(ext_own, 0, kv_len) : 0;
    hi = lo + mp_clamp(ext_all, 0, kv_len);           // the item's last token sees the most
  }
#else
  const int req = blockIdx.x;
  const int lo = mp_clamp(CL_ARG_INDPTR[req], 0, n_idx);
  int hi = mp_clamp(CL_ARG_INDPTR[req + 1], 0, n_idx);
  hi = hi > lo ? hi : lo;
#endif
#if CL_PREFILL
  const int n_tok = n_tok_own;                        // keys this wave's token weighs
  const int n_steps = __builtin_amdgcn_readfirstlane((hi - lo + MP_STEP - 1) / MP_STEP);   // steps of the item (the same for all its waves)
#else
  const int n_tok = hi - lo;
  const int n_steps = __builtin_amdgcn_readfirstlane((n_tok + MP_STEP - 1) / MP_STEP);
#endif
  const float scale_log2e = sm_scale * 1.4426950408889634f;
#if CL_PREFILL
  const i64 qrow = (i64)qtok * CL_HEADS + head0 + c;
#else
  const i64 qrow = (i64)req * CL_HEADS + head0 + c;
#endif
  elem_t* my_tiles = mp_tiles + kw * (CL_MP_STAGES * MP_TILE);     // (key-sharing waves: images of one's own)
  const unsigned tiles_byte = (unsigned)(size_t)(__attribute__((address_space(3))) elem_t*)my_tiles;

  float m_run = CL_NEG_BIG;            // softmax reference point of head c (log2 domain), uniform over g
  f32x4 l_acc = {0.f, 0.f, 0.f, 0.f};  // every component: sum of the (element-typed) weights of head c: normalises out
  float l_exact = 0.f;                 // this lane's share of the sum of the unrounded weights: the lse (a row
                                       // with a handful of keys would show the rounding in its lse otherwise)
  f32x4 acc[MP_FB];                    // acc[fb][r] = O[head c][16 fb + 4 g + r]
#pragma unroll
  for (int fb = 0; fb < MP_FB; ++fb) acc[fb] = (f32x4){0.f, 0.f, 0.f, 0.f};

  if (n_steps > 0) {
    elem8 ones;
#pragma unroll
    for (int i = 0; i < 8; ++i) ones[i] = to_elem(1.0f);

    // table entries of a 256-entry window: register k holds entry 64 k + lane (positions past the
    // item's end repeat its last entry; ids outside the pool are clamped into it where they are
    // used, not here: touching a loaded value waits for it, and with it for every row asked for
    // before it)
    auto load_window = [&](int w, int (&ids)[4]) __attribute__((always_inline)) {
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        int pos = lo + w * MP_WINDOW + 64 * k + lane;
        pos = pos < hi - 1 ? pos : hi - 1;
        ids[k] = CL_ARG_INDICES[pos];
      }
    };
    // `ids_cur`: the entries of window `cur_window`, the one the rows asked for next are in;
    // `ids_next`: those of the window after it, asked for when `ids_cur` was taken up
    int ids_cur[4], ids_next[4];
    int cur_window = 0;
    load_window(0, ids_cur);
    if (MP_WINDOW < hi - lo) {
      load_window(1, ids_next);
    } else {
#pragma unroll
      for (int k = 0; k < 4; ++k) ids_next[k] = ids_cur[k];
    }

    // the rows of step s into this wave's image `image`: lane l loads token row 8 rg + l / 8 of the
    // step (its table entry fetched from the lane of `ids_cur` that holds it), the chunk that belongs
    // in slot l % 8 of that row.  Steps are asked for in rising order; stepping into the next
    // window takes its entries up and asks for those of the one after.
    auto issue_step = [&](int s, int image) __attribute__((always_inline)) {
      if (s / (MP_WINDOW / MP_STEP) != cur_window) {
        cur_window = s / (MP_WINDOW / MP_STEP);
#pragma unroll
        for (int k = 0; k < 4; ++k) ids_cur[k] = ids_next[k];
        if ((cur_window + 1) * MP_WINDOW < hi - lo) load_window(cur_window + 1, ids_next);
      }
      const int in_window = s % (MP_WINDOW / MP_STEP);
      const int k = in_window >> 1;
      const int held = k == 0 ? ids_cur[0] : k == 1 ? ids_cur[1] : k == 2 ? ids_cur[2] : ids_cur[3];
      const unsigned stage_byte = tiles_byte + (unsigned)(image * MP_TILE * 2);
#pragma unroll
      for (int i = 0; i < 4 / MP_SHARE; ++i) {
        const int rg = tw * (MP_SHARE > 1) + i * MP_SHARE;   // (the waves of a shared image divide a step's four row groups)
        const int r = 8 * rg + (lane >> 3);
        const int src_lane = 32 * (in_window & 1) + r;
        const int id = mp_clamp(__builtin_amdgcn_ds_bpermute(src_lane << 2, held), 0, num_pages - 1);
        const int chunk = (lane & 7) ^ mp_swz(r);
        const char* lat_src = reinterpret_cast<const char*>(CL_ARG_KV) + ((i64)id * CL_CKV + 8 * chunk) * 2;
        const char* pe_src = reinterpret_cast<const char*>(CL_ARG_KPE) + ((i64)id * CL_KPE + 8 * chunk) * 2;
        mp_issue_row_group<0>(lat_src, pe_src, stage_byte + (unsigned)(rg * 1024));
      }
    };
#pragma unroll
    for (int i = 0; i < MP_AHEAD; ++i)
      if (kw + i * MP_KS < n_steps) issue_step(kw + i * MP_KS, i);

    // Q fragments (B operand of the score product): lane (c, g) holds q[head c][32 j + 8 g .. +8]
    elem8 qf[MP_KJ];
#pragma unroll
    for (int j = 0; j < MP_KJ; ++j) {
      const int col = 32 * j + 8 * g;
      const elem_t* src = col < CL_CKV ? CL_ARG_Q + qrow * CL_CKV + col : CL_ARG_QPE + qrow * CL_KPE + (col - CL_CKV);
      qf[j] = as_elem8(ld16(src));
    }
    // (the wait for the Q fragments belongs here, once: left to their first use it would sit in the
    // loop, where it waits for every row in flight at every step)
#pragma unroll
    for (int j = 0; j < MP_KJ; ++j) asm volatile("" :: "v"(qf[j]));

    // this lane's operand offsets inside an image (elements):
    //   score operand: token row c of a 16-token half, chunk g of a 32-feature block
    //   value operand: its 8-byte piece of the 4 (token) x 16 (feature) patch of lane group g
    const int a_lo = c * 64 + ((g ^ mp_swz(c)) << 3);
    const int vtok = 4 * g + (c >> 2);
    const int v_lo = vtok * 64 + (((((c & 3) >> 1)) ^ mp_swz(vtok)) << 3) + 4 * (c & 1);

    // Softmax as in the dense kernel: weights are exp2(score - m_run) against a fixed reference,
    // row sums by one more matrix op against ones, nothing crosses lanes in the hot loop; a
    // score more than MP_RESCALE_STEP above the reference leaves the loop before the step is
    // consumed, the cold block raises the reference, rescales (l, O) and re-enters at the step.
    int step = kw;                     // this wave's steps: kw, kw + MP_KS, ..
    int image = 0;                     // the image `step` is in: its number among this wave's steps, modulo the images
    bool front_done = false;           // the loads of `step` have been waited for and the next ones issued
    for (;;) {
      bool raise_any = false;
      float mxl = CL_NEG_BIG;
      while (step < n_steps) {
        if (!front_done) {
          // The rows of `step` have landed when only what was asked for after them is on its way:
          // the rows of the steps behind it that the item has, at most MP_AHEAD - 1 of them (loads
          // land in the order they were asked for; table entries read a window ahead lie between
          // and only make the wait stricter).  The barrier makes that everybody's share, and says
          // that everybody is done with the image of step - 1, which the rows of step + MP_AHEAD
          // go into (key-sharing waves have images of their own and no barrier).
          {
            const int behind = (n_steps - 1 - step) / MP_KS;       // steps of this wave's behind `step`
            if (MP_AHEAD >= 3 && behind >= 2) {
              MP_WAITCNT(2 * MP_UNITS);
            } else if (MP_AHEAD >= 2 && behind >= 1) {
              MP_WAITCNT(MP_UNITS);
            } else {
              MP_WAITCNT(0);
            }
          }
          if (MP_SHARE > 1) __syncthreads();
          if (step + MP_AHEAD * MP_KS < n_steps) issue_step(step + MP_AHEAD * MP_KS, (image + MP_AHEAD) % CL_MP_STAGES);
          front_done = true;
        }
        const elem_t* tile = my_tiles + image * MP_TILE;
#if CL_PREFILL
        // a wave whose token sees none of this step's keys (or that has no token: it only helps
        // load) leaves the images to the waves that need them
        if (step * MP_STEP >= n_tok) {
          step += MP_KS;
          image = (image + 1) % CL_MP_STAGES;
          front_done = false;
          continue;
        }
#endif

        // scores^T: rows = tokens 16 h + (0..15), columns = heads
        f32x4 st[2];
        st[0] = st[1] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < MP_KJ; ++j) {
#pragma unroll
          for (int h = 0; h < 2; ++h) {
            const elem8 a = *reinterpret_cast<const elem8*>(tile + (j >> 1) * MP_PANEL + 16 * h * 64 +
                                                            (a_lo ^ ((4 * (j & 1)) << 3)));
            st[h] = mfma16(a, qf[j], st[h]);
          }
        }
        __builtin_amdgcn_sched_group_barrier(0x100, CL_LDS_AHEAD, 0);
#pragma unroll
        for (int n = 0; n < 2 * MP_KJ - CL_LDS_AHEAD; ++n) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
        __builtin_amdgcn_sched_group_barrier(0x008, CL_LDS_AHEAD, 0);

        // scaled scores; tokens past the item's end weigh nothing
        const int t0 = step * MP_STEP;
        float v = CL_NEG_BIG;
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            st[h][r] = t0 + 16 * h + 4 * g + r < n_tok ? st[h][r] * scale_log2e : CL_NEG_BIG;
            v = fmaxf(v, st[h][r]);
          }
        mxl = v;
        if (step == kw && m_run < 0.5f * CL_NEG_BIG) {
          // first step (nothing accumulated yet): its own maximum is the reference
          float mx = mxl;
          mx = fmaxf(mx, lane_xor(mx, lane, 16));
          mx = fmaxf(mx, lane_xor(mx, lane, 32));
          m_run = mx;
        } else if (__builtin_amdgcn_ballot_w64(mxl > m_run + MP_RESCALE_STEP)) {   // wave-uniform
          raise_any = true;
          break;
        }

        elem8 pf;
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
          for (int r = 0; r < 4; ++r) {
#if CL_PREFILL
            // (a wave whose token sees none of a step's keys has no reference yet: test the mask itself)
            const float p = st[h][r] > 0.5f * CL_NEG_BIG ? fast_exp2(st[h][r] - m_run) : 0.f;
#else
            const float p = fast_exp2(st[h][r] - m_run);
#endif
            l_exact += p;
            pf[4 * h + r] = to_elem(p);
          }

        // out^T block fb: rows = features 16 fb + (0..15), slots = tokens 4 g + (0..3), 16 + 4 g + (0..3)
        l_acc = mfma16(ones, pf, l_acc);
#pragma unroll
        for (int fb = 0; fb < MP_FB; ++fb) {
          const elem_t* p = tile + (fb >> 2) * MP_PANEL + (v_lo ^ (((2 * fb) & 7) << 3));
          const mp_s16x4 lo4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((mp_lds_s16x4*)(p));
          const mp_s16x4 hi4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((mp_lds_s16x4*)(p + 16 * 64));
          const elem8 a = __builtin_bit_cast(elem8, (mp_s16x8)__builtin_shufflevector(lo4, hi4, 0, 1, 2, 3, 4, 5, 6, 7));
          acc[fb] = mfma16(a, pf, acc[fb]);
        }
        __builtin_amdgcn_sched_group_barrier(0x100, CL_LDS_AHEAD, 0);
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
#pragma unroll
        for (int n = 0; n < MP_FB - CL_LDS_AHEAD / 2; ++n) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
        }
        __builtin_amdgcn_sched_group_barrier(0x008, CL_LDS_AHEAD / 2, 0);

        step += MP_KS;
        image = (image + 1) % CL_MP_STAGES;
        front_done = false;
      }
      if (!raise_any) break;
      // cold: raise the reference and rescale what has been accumulated
      float mx = mxl;
      mx = fmaxf(mx, lane_xor(mx, lane, 16));
      mx = fmaxf(mx, lane_xor(mx, lane, 32));
      const bool up = mx > m_run + MP_RESCALE_STEP;
      const float m_new = up ? mx : m_run;
      const float alpha = up ? fast_exp2(m_run - m_new) : 1.0f;
      m_run = m_new;
      l_acc *= alpha;
      l_exact *= alpha;
#pragma unroll
      for (int fb = 0; fb < MP_FB; ++fb) acc[fb] *= alpha;
    }
    // (no load is on its way into LDS any more: the last step's wait left none)
    __builtin_amdgcn_s_waitcnt(0x0F70);
  }

#if MP_KS > 1
  // ---- the key-sharing waves fold into the first --------------------------------------------------
  // Every other wave leaves (accumulators, reference point, sums) in its first image as they lie in
  // its registers -- nothing reads that image any more and no load is on its way into it -- and
  // the first wave folds them into its own by the max-rescale rule (a wave that had no step stands
  // at the lowest reference point with sums of zero).
  {
    constexpr int sums_at = MP_FB * 64 * 4;
    if (kw > 0) {
      float* park = reinterpret_cast<float*>(my_tiles);
#pragma unroll
      for (int fb = 0; fb < MP_FB; ++fb) *reinterpret_cast<f32x4*>(park + (fb * 64 + lane) * 4) = acc[fb];
      park[sums_at + lane] = m_run;
      park[sums_at + 64 + lane] = l_acc[0];
      park[sums_at + 128 + lane] = l_exact;
    }
    __syncthreads();
    if (kw > 0) return;
#pragma unroll
    for (int w = 1; w < MP_KS; ++w) {
      const float* theirs = reinterpret_cast<const float*>(mp_tiles + w * (CL_MP_STAGES * MP_TILE));
      const float m_o = theirs[sums_at + lane];
      const float m_new = fmaxf(m_run, m_o);
      const float a = fast_exp2(m_run - m_new), b = fast_exp2(m_o - m_new);
      m_run = m_new;
      l_acc = l_acc * a + theirs[sums_at + 64 + lane] * b;
      l_exact = l_exact * a + theirs[sums_at + 128 + lane] * b;
#pragma unroll
      for (int fb = 0; fb < MP_FB; ++fb)
        acc[fb] = acc[fb] * a + *reinterpret_cast<const f32x4*>(theirs + (fb * 64 + lane) * 4) * b;
    }
  }
#endif

  // ---- write this wave's heads ------------------------------------------------------------------
#if CL_PREFILL
  if (!tok_live) return;
#endif
  const float l = l_acc[0];
  const int f0 = 4 * g;
#if CL_CHUNKED
  // The partial sum that leaves is the one of the unrounded weights: the combined lse is read from
  // it, and it normalises the combined output as the reference's kernels do (against the sum of
  // the rounded weights the output differs by less than its own rounding; rescaling the
  // accumulators to match cost a lone wave 128 multiplies, half a microsecond per item).
  const i64 prow = (i64)item * CL_HEADS + head0 + c;
  l_exact += lane_xor(l_exact, lane, 16);
  l_exact += lane_xor(l_exact, lane, 32);
  (void)l;
#pragma unroll
  for (int fb = 0; fb < MP_FB; ++fb)
    *reinterpret_cast<f32x4*>(CL_ARG_PO + prow * CL_CKV + f0 + 16 * fb) = acc[fb];
  if (g == 0) {
    CL_ARG_PM[prow] = m_run;
    CL_ARG_PL[prow] = l_exact;
  }
#else
  // an empty request has l == 0: the floor turns 0/0 into 0 and its lse is -inf
  const float inv = 1.0f / fmaxf(l, 1.0e-30f);
  elem_t* dst_row = CL_ARG_OUT + qrow * CL_CKV;
#if CL_EMIT_LSE
  l_exact += lane_xor(l_exact, lane, 16);
  l_exact += lane_xor(l_exact, lane, 32);
  if (g == 0) CL_ARG_LSE[qrow] = l_exact > 0.f ? m_run + fast_log2(l_exact) : CL_NEG_INF;
#endif
  // A lane holds features 16 fb + 4 g .. + 3 of its head for every block fb.  Lanes g and g ^ 1
  // trade halves of a pair of blocks (one row swap per register), so that each stores 16
  // contiguous bytes: even g the 8 features from 4 g of the even block, odd g those from
  // 4 (g - 1) of the odd one (as 8-byte pieces the 32 stores of a wave took over a microsecond).
  (void)f0;
  elem_t* dst = dst_row + 16 * (g & 1) + 4 * (g & 2);
#pragma unroll
  for (int fp = 0; fp < MP_FB / 2; ++fp) {
    elem4 y0, y1;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      y0[r] = to_elem(acc[2 * fp][r] * inv);
      y1[r] = to_elem(acc[2 * fp + 1][r] * inv);
    }
    const u32x2 a = __builtin_bit_cast(u32x2, y0), b = __builtin_bit_cast(u32x2, y1);
    unsigned a0 = a[0], a1 = a[1], b0 = b[0], b1 = b[1];
    mp_swap_rows16(a0, b0);
    mp_swap_rows16(a1, b1);
    *reinterpret_cast<u32x4*>(dst + 32 * fp) = (u32x4){a0, a1, b0, b1};
  }
#endif
}
#endif  // CL_EMIT_PARTIAL
