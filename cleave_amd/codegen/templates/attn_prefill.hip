// ---- causal prefill attention (GQA), ragged queries; keys/values through a token table
// (page size 1) or packed per request ---------------------------------------------------------
//
//   out[q] = softmax(mask(Q[q] K^T * sm_scale)) V,   keep kv_pos <= kv_len - q_len + q_pos
//
// Queries of all requests are packed (total_q, q_heads, d) with qo_indptr; a request's keys are
// the rows its slice of the token table names (cache (num_pages, 1, kv_heads, d)), or with
// CL_RAGGED rows kv_indptr[r] .. kv_indptr[r+1] of packed K / V (total_kv, kv_heads, d).
//
// Work items: a query tile holds 16 rows = PF_TOK query tokens x the head group of one kv head
// (the matrix-op N extent); an item is the tile of at most PF_TOK consecutive tokens of one
// request, a new item at every multiple of PF_TOK packed tokens and at every request boundary
// (item t = chunk w + request b for the one pair that overlaps, as in the chunked decode).  A
// workgroup holds one wave per kv head, so its waves together read whole token rows of the
// cache.  Per wave the arithmetic is the decode kernel's: K rows are the A operand as loaded
// (scores^T = K Q^T), V is transposed 8x8 in registers, out^T += V^T P^T takes P^T from the
// score registers in place, online softmax lane-local per query row.  The causal limit of a row
// is a per-lane constant compared with the token index of each score; an item stops at the last
// key any of its rows may see.  Rows no key is kept for give 0 and lse -inf.
//
//   CL_HEAD_DIM (= value width, multiple of 128 or 64)  CL_KV_HEADS  CL_Q_HEADS  CL_RAGGED
//   run-time: batch, total_q, n_idx (table length / total_kv), num_pages (table form), sm_scale

#define PF_STEP 32
#define PF_GROUP (CL_Q_HEADS / CL_KV_HEADS)
#define PF_TOK (16 / PF_GROUP)                 // query tokens per item
#define PF_KJ (CL_HEAD_DIM / 32)
#define PF_VC ((CL_HEAD_DIM + 127) / 128)
static_assert(CL_Q_HEADS % CL_KV_HEADS == 0 && 16 % PF_GROUP == 0, "the head group divides the 16-row query tile");
static_assert(CL_HEAD_DIM % 32 == 0 && (CL_HEAD_DIM % 128 == 0 || CL_HEAD_DIM == 64), "head dim 64 or k*128");

struct PfTile {                // one 32-token step's K and V, as loaded
  u32x4 k[2][PF_KJ];
  u32x4 v[PF_VC][8];
};

CL_DEVICE int pf_clamp(int v, int lo, int hi) { return v < lo ? lo : (v > hi ? hi : v); }
template <int V> struct PfC { static constexpr int value = V; };

#if CL_EMIT_PARTIAL
extern "C" __global__ void __launch_bounds__(CL_KV_HEADS * 64)
CL_PARTIAL_NAME(CL_PARTIAL_PARAMS) {
  const int lane = threadIdx.x & 63, head = threadIdx.x >> 6;
  const int c = lane & 15, g = lane >> 4;
  const int item = blockIdx.x;
  // the request whose items include `item`: the last b with b + qo_indptr[b] / PF_TOK <= item
  const ClRequest found = cl_find_request(CL_ARG_QINDPTR, batch, total_q, PF_TOK, 1, item, lane, CL_ARG_INDPTR, n_idx);
  const int req = found.req, q0 = found.p0, q1 = found.p1;
  const int chunk = item - req;
  const int lo = q0 > chunk * PF_TOK ? q0 : chunk * PF_TOK;
  const int hi = q1 < (chunk + 1) * PF_TOK ? q1 : (chunk + 1) * PF_TOK;
  if (hi <= lo) return;                                 // an index no (chunk, request) pair maps to
  const int kv0 = found.s0;
  int kv_len = found.s1 - kv0;
  kv_len = kv_len > 0 ? kv_len : 0;
  const int off = kv_len - (q1 - q0);                   // key position of the request's first query row
  const int n_rows = (hi - lo) * PF_GROUP;
  // this lane's query row (column c of the score tile): token, head, last key it may see
  const bool live = c < n_rows;
  const int tok = lo + (live ? c / PF_GROUP : 0);
  const int qhead = head * PF_GROUP + (live ? c % PF_GROUP : 0);
  const int limit = live ? off + (tok - q0) : -1;
  int ext = off + (hi - 1 - q0) + 1;                    // keys the item's last row may see
  ext = ext < kv_len ? ext : kv_len;
  ext = ext > 0 ? ext : 0;
  if (ext == 0) {
    // no row of the item sees a key (a key window shorter than the query run leaves whole tiles
    // like this): zeros and -inf, nothing to read
    for (int idx = lane; idx < n_rows * (CL_HEAD_DIM / 4); idx += 64) {
      const int row = idx / (CL_HEAD_DIM / 4), d = (idx % (CL_HEAD_DIM / 4)) * 4;
      const i64 orow = (i64)(lo + row / PF_GROUP) * CL_Q_HEADS + head * PF_GROUP + row % PF_GROUP;
      elem4 y;
#pragma unroll
      for (int i = 0; i < 4; ++i) y[i] = to_elem(0.f);
      *reinterpret_cast<elem4*>(CL_ARG_OUT + orow * CL_HEAD_DIM + d) = y;
    }
#if CL_EMIT_LSE
    if (g == 0 && live) CL_ARG_LSE[(i64)tok * CL_Q_HEADS + qhead] = CL_NEG_INF;
#endif
    return;
  }
  const float scale2 = sm_scale * 1.4426950408889634f;
  const i64 row_stride = (i64)CL_KV_HEADS * CL_HEAD_DIM;
  const elem_t* kbase = CL_ARG_K + (i64)head * CL_HEAD_DIM;
  const elem_t* vbase = CL_ARG_V + (i64)head * CL_HEAD_DIM;
  const int n_steps = (ext + PF_STEP - 1) / PF_STEP;
  const int last_step = n_steps > 0 ? n_steps - 1 : 0;

  // Query rows as the B operand: lane (c, g) holds Q[row c][32 j + 8 g .. +8]; padded rows are 0.
  elem8 qf[PF_KJ];
  {
    const elem_t* row = CL_ARG_Q + ((i64)tok * CL_Q_HEADS + qhead) * CL_HEAD_DIM + 8 * g;
#pragma unroll
    for (int j = 0; j < PF_KJ; ++j) {
      u32x4 raw = ld16(row + 32 * j);
      if (!live) raw = (u32x4){0u, 0u, 0u, 0u};
      qf[j] = as_elem8(raw);
    }
  }

  float m_run = CL_NEG_BIG;   // running max of the scaled scores (log2 domain), uniform over g
  float l_run = 0.f;          // this lane's share of the running sum of the rounded weights (normalises out)
  float l_exact = 0.f;        // ... of the unrounded ones (the lse)
  f32x4 acc[PF_VC][8];        // acc[vc][j][r] = O[row c][128 vc + 32 g + 8 r + j]
#pragma unroll
  for (int vc = 0; vc < PF_VC; ++vc)
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[vc][j] = (f32x4){0.f, 0.f, 0.f, 0.f};

  if (n_steps > 0) {
    // Row of key position t of this request (clamped onto the item's last key: scores past it are
    // masked).  Table form: lane i of `ids` holds the table entry of key 32 s + (i % 32) of
    // step s, read one step before the rows it names.
#if !CL_RAGGED
    auto load_ids = [&](int s) __attribute__((always_inline)) -> int {
      s = s < last_step ? s : last_step;
      int t = s * PF_STEP + (lane & 31);
      t = t < ext - 1 ? t : ext - 1;
      return pf_clamp(CL_ARG_INDICES[kv0 + t], 0, num_pages - 1);
    };
#endif
    auto load_tile = [&](int s, int ids, PfTile& tile) __attribute__((always_inline)) {
      s = s < last_step ? s : last_step;
      const int t0 = s * PF_STEP;
      auto row_of = [&](int t) __attribute__((always_inline)) -> i64 {
        t = t < ext - 1 ? t : ext - 1;
#if CL_RAGGED
        (void)ids;
        return (i64)(kv0 + t) * row_stride;
#else
        return (i64)__builtin_amdgcn_ds_bpermute((t - t0) << 2, ids) * row_stride;
#endif
      };
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const elem_t* row = kbase + row_of(t0 + 16 * h + c) + 8 * g;
#pragma unroll
        for (int j = 0; j < PF_KJ; ++j) tile.k[h][j] = ld16(row + 32 * j);
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const elem_t* row = vbase + row_of(t0 + (e < 4 ? 4 * g + e : 16 + 4 * g + (e - 4)));
#pragma unroll
        for (int vc = 0; vc < PF_VC; ++vc) {
          int col = 128 * vc + 8 * c;
          if (CL_HEAD_DIM % 128 != 0) col = col < CL_HEAD_DIM - 8 ? col : CL_HEAD_DIM - 8;
          tile.v[vc][e] = ld16(row + col);
        }
      }
    };

    // Two register tiles: while step n is in the matrix cores the loads of step n + 1 are in
    // flight.  The loop runs whole turns of the pair whose next steps both exist, with no branch
    // in its body (with one, the waits placed at the loop head had to assume that loads of the
    // part branched around were still on their way, and waited for the current tile before asking
    // for the next); the last one or two steps follow as straight-line code that asks for nothing
    // past the item's last step.
    PfTile ring[2];
    int ids_next = 0;
#if !CL_RAGGED
    {
      const int ids_first = load_ids(0);
      ids_next = load_ids(1);
      load_tile(0, ids_first, ring[0]);
    }
#else
    load_tile(0, 0, ring[0]);
#endif
    auto one_step = [&](auto r_c, const int step, const bool ask) __attribute__((always_inline)) {
      constexpr int r = decltype(r_c)::value;
      {
        if (ask) {
          // (the table entries of the step after next are asked for ahead of the next step's rows:
          // loads land in the order they were asked for, so waiting for entries asked for behind
          // the rows would wait for the rows)
#if !CL_RAGGED
          const int ids_after = load_ids(step + 2);
          load_tile(step + 1, ids_next, ring[r ^ 1]);
          ids_next = ids_after;
#else
          load_tile(step + 1, ids_next, ring[r ^ 1]);
#endif
        }
        const PfTile& cur = ring[r];
        const int t0 = step * PF_STEP;

        // scores^T for the two 16-token halves
        float s[8];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          f32x4 st = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int j = 0; j < PF_KJ; ++j) st = mfma16(as_elem8(cur.k[h][j]), qf[j], st);
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const int t = t0 + 16 * h + 4 * g + q;
            s[4 * h + q] = (t < ext && t <= limit) ? st[q] * scale2 : CL_NEG_BIG;
          }
        }
        float mx = s[0];
#pragma unroll
        for (int i = 1; i < 8; ++i) mx = fmaxf(mx, s[i]);
        mx = fmaxf(mx, lane_xor(mx, lane, 16));
        mx = fmaxf(mx, lane_xor(mx, lane, 32));
        const float m_new = fmaxf(m_run, mx);
        const float alpha = fast_exp2(m_run - m_new);
        m_run = m_new;
        elem8 pf;
        float psum = 0.f, esum = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          // masked slots hold CL_NEG_BIG; when the whole row is still masked m_new equals it too,
          // so test the mask itself rather than trusting exp2 of a zero difference
          float p = s[i] > 0.5f * CL_NEG_BIG ? fast_exp2(s[i] - m_new) : 0.f;
          elem_t pe = to_elem(p);
          psum += to_f32(pe);            // the normalising sum uses the weights the value product really sees
          esum += p;                     // (a row with a handful of keys shows the rounding in its lse otherwise)
          pf[i] = pe;
        }
        l_run = l_run * alpha + psum;
        l_exact = l_exact * alpha + esum;
        if (__builtin_amdgcn_ballot_w64(alpha != 1.0f)) {   // wave-uniform: skip when no max moved
#pragma unroll
          for (int vc = 0; vc < PF_VC; ++vc)
#pragma unroll
            for (int j = 0; j < 8; ++j) acc[vc][j] *= alpha;
        }
#pragma unroll
        for (int vc = 0; vc < PF_VC; ++vc) {
          u32x4 vt[8];
          transpose8x8(cur.v[vc], vt);
#pragma unroll
          for (int j = 0; j < 8; ++j) acc[vc][j] = mfma16(as_elem8(vt[j]), pf, acc[vc][j]);
        }
      }
    };
    int base = 0;
    for (; base + 2 < n_steps; base += 2) {
      one_step(PfC<0>{}, base, true);
      one_step(PfC<1>{}, base + 1, true);
    }
    if (base < n_steps) one_step(PfC<0>{}, base, base + 1 < n_steps);
    if (base + 1 < n_steps) one_step(PfC<1>{}, base + 1, false);
  }

  // ---- each lane writes its row's features straight from the accumulators, 16 bytes at a time ----
  // (acc[vc][0..7][r] are the eight consecutive features 128 vc + 32 g + 8 r .. of row c)
  l_run += lane_xor(l_run, lane, 16);
  l_run += lane_xor(l_run, lane, 32);
  l_exact += lane_xor(l_exact, lane, 16);
  l_exact += lane_xor(l_exact, lane, 32);
  if (!live) return;
  const float inv = 1.0f / fmaxf(l_run, 1.0e-30f);            // a row with no key: 0 and lse -inf
  elem_t* dst = CL_ARG_OUT + ((i64)tok * CL_Q_HEADS + qhead) * CL_HEAD_DIM;
#pragma unroll
  for (int vc = 0; vc < PF_VC; ++vc)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int d = 128 * vc + 32 * g + 8 * r;
      if (CL_HEAD_DIM % 128 != 0 && d >= CL_HEAD_DIM) continue;
      elem8 y;
#pragma unroll
      for (int j = 0; j < 8; ++j) y[j] = to_elem(acc[vc][j][r] * inv);
      st16(dst + d, as_u32x4(y));
    }
#if CL_EMIT_LSE
  if (g == 0) CL_ARG_LSE[(i64)tok * CL_Q_HEADS + qhead] = l_exact > 0.f ? m_run + fast_log2(l_exact) : CL_NEG_INF;
#endif
}
#endif  // CL_EMIT_PARTIAL
