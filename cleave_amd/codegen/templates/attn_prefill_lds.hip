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
// stages rotate (two steps of loads in flight), one barrier per step; the softmax is the exact
// online one of the decode kernel, lane-local per query row.
//
// Work items: a new item at every multiple of PL_QT packed query tokens and at every request
// boundary (item t = chunk w + request b for the one pair that overlaps); an item stops at the
// last key any of its rows may see and writes zeros / -inf without reading when it sees none.
//
//   CL_HEAD_DIM (multiple of 64)  CL_KV_HEADS  CL_Q_HEADS (group divides 16)  CL_RAGGED
//   run-time: batch, total_q, n_idx (table length / total_kv), num_pages (table form), sm_scale

#define PL_STEP 32
#define PL_GROUP (CL_Q_HEADS / CL_KV_HEADS)
#define PL_ROWS 128
#define PL_QT (PL_ROWS / PL_GROUP)            // query tokens per item
#define PL_PANELS (CL_HEAD_DIM / 64)
#define PL_PANEL (PL_STEP * 64)               // elements of one 64-feature panel
#define PL_IMG (PL_PANELS * PL_PANEL)         // elements of one operand image
#define PL_STAGE (2 * PL_IMG)                 // K image, then V image
#define PL_STAGES 3
#define PL_KJ (CL_HEAD_DIM / 32)
#define PL_FB (CL_HEAD_DIM / 16)
#define PL_UNITS_PER (2 * PL_PANELS)          // 1 KiB loads per wave and step: its 8-key group of every panel of K and V
#define PL_WINDOW 256                         // table entries held in registers at a time
static_assert(CL_Q_HEADS % CL_KV_HEADS == 0 && 16 % PL_GROUP == 0, "the head group divides the 16-row query tile");
static_assert(CL_HEAD_DIM % 64 == 0 && CL_HEAD_DIM <= 256, "head dim in whole 64-feature panels");
static_assert(PL_UNITS_PER < 16, "load counter range");

__shared__ __attribute__((aligned(1024))) elem_t pl_tiles[PL_STAGES * PL_STAGE];

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
               :: "v"(gptr), "s"(__builtin_amdgcn_readfirstlane(lds_byte)), "n"(OFF) : "memory");
}
template <int P>
CL_DEVICE void pl_issue_panels(const char* src, unsigned group_byte) {
  if constexpr (P < PL_PANELS) {
    pl_dma16<128 * P>(src, group_byte + (unsigned)(P * PL_PANEL * 2) - 128 * P);
    pl_issue_panels<P + 1>(src, group_byte);
  }
}

#if CL_EMIT_PARTIAL
extern "C" __global__ void __launch_bounds__(256, 2)
CL_PARTIAL_NAME(CL_PARTIAL_PARAMS) {
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int c = lane & 15, g = lane >> 4;
  const int item = blockIdx.x, head = blockIdx.y;
  // the request whose items include `item`: the last b with b + qo_indptr[b] / PL_QT <= item
  int req = 0;
  {
    int hi_b = batch - 1;
    while (req < hi_b) {
      const int mid = (req + hi_b + 1) >> 1;
      if (mid + pl_clamp(CL_ARG_QINDPTR[mid], 0, total_q) / PL_QT <= item) req = mid;
      else hi_b = mid - 1;
    }
  }
  const int q0 = pl_clamp(CL_ARG_QINDPTR[req], 0, total_q), q1 = pl_clamp(CL_ARG_QINDPTR[req + 1], 0, total_q);
  const int chunk = item - req;
  const int lo = q0 > chunk * PL_QT ? q0 : chunk * PL_QT;
  const int hi = q1 < (chunk + 1) * PL_QT ? q1 : (chunk + 1) * PL_QT;
  if (hi <= lo) return;                                 // an index no (chunk, request) pair maps to
  const int kv0 = pl_clamp(CL_ARG_INDPTR[req], 0, n_idx);
  int kv_len = pl_clamp(CL_ARG_INDPTR[req + 1], 0, n_idx) - kv0;
  kv_len = kv_len > 0 ? kv_len : 0;
  const int off = kv_len - (q1 - q0);                   // key position of the request's first query row
  const int n_rows = (hi - lo) * PL_GROUP;
  int ext = off + (hi - 1 - q0) + 1;                    // keys the item's last row may see
  ext = ext < kv_len ? ext : kv_len;
  ext = ext > 0 ? ext : 0;

  // this lane's two query rows (column c of each of the wave's score tiles): token, head, last key it may see
  bool live[2];
  int tok[2], qhead[2], limit[2];
#pragma unroll
  for (int rt = 0; rt < 2; ++rt) {
    const int m = 32 * wave + 16 * rt + c;
    live[rt] = m < n_rows;
    tok[rt] = lo + (live[rt] ? m / PL_GROUP : 0);
    qhead[rt] = head * PL_GROUP + (live[rt] ? m % PL_GROUP : 0);
    limit[rt] = live[rt] ? off + (tok[rt] - q0) : -1;
  }

  if (ext == 0) {
    // no row of the item sees a key: zeros and -inf, nothing to read
#pragma unroll
    for (int rt = 0; rt < 2; ++rt) {
      if (!live[rt]) continue;
      elem_t* dst = CL_ARG_OUT + ((i64)tok[rt] * CL_Q_HEADS + qhead[rt]) * CL_HEAD_DIM + 4 * g;
      elem4 z;
#pragma unroll
      for (int i = 0; i < 4; ++i) z[i] = to_elem(0.f);
#pragma unroll
      for (int fb = 0; fb < PL_FB; ++fb) *reinterpret_cast<elem4*>(dst + 16 * fb) = z;
#if CL_EMIT_LSE
      if (g == 0) CL_ARG_LSE[(i64)tok[rt] * CL_Q_HEADS + qhead[rt]] = CL_NEG_INF;
#endif
    }
    return;
  }

  const float scale2 = sm_scale * 1.4426950408889634f;
  const i64 row_bytes = (i64)CL_KV_HEADS * CL_HEAD_DIM * 2;
  const char* kbase = reinterpret_cast<const char*>(CL_ARG_K) + (i64)head * CL_HEAD_DIM * 2;
  const char* vbase = reinterpret_cast<const char*>(CL_ARG_V) + (i64)head * CL_HEAD_DIM * 2;
  const int n_steps = (ext + PL_STEP - 1) / PL_STEP;
  const unsigned tiles_byte = (unsigned)(size_t)(__attribute__((address_space(3))) elem_t*)pl_tiles;

  // Table entries of a 256-key window: register k holds the entry of key 256 w + 64 k + lane
  // (positions past the item's last key repeat it; ids outside the pool are clamped into it).
#if !CL_RAGGED
  auto load_window = [&](int w, int (&ids)[4]) __attribute__((always_inline)) {
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      int t = w * PL_WINDOW + 64 * k + lane;
      t = t < ext - 1 ? t : ext - 1;
      ids[k] = pl_clamp(CL_ARG_INDICES[kv0 + t], 0, num_pages - 1);
    }
  };
  int ids_cur[4], ids_next[4];     // the window the loads are in, and the one after it
  load_window(0, ids_cur);
  load_window(1, ids_next);        // (clamped onto the last key when there is no second window)
#endif
  // This wave's share of step s (clamped onto the last step: a step past the end reloads the last
  // one into an image nobody reads, so the load counter holds the same number of steps at every
  // wait): key rows 8 wave + lane / 8 of every panel of K and V, the chunk for slot lane % 8.
  auto issue_step = [&](int s, int slot) __attribute__((always_inline)) {
    s = s < n_steps - 1 ? s : n_steps - 1;
    const int r = 8 * wave + (lane >> 3);
    int t = s * PL_STEP + r;
    t = t < ext - 1 ? t : ext - 1;
#if CL_RAGGED
    const i64 row = (i64)(kv0 + t);
#else
    const int in_window = s % (PL_WINDOW / PL_STEP);
    const int k = in_window >> 1;
    const int held = k == 0 ? ids_cur[0] : k == 1 ? ids_cur[1] : k == 2 ? ids_cur[2] : ids_cur[3];
    const i64 row = __builtin_amdgcn_ds_bpermute((t - (s - in_window) * PL_STEP - 64 * k) << 2, held);
#endif
    const int chunk = (lane & 7) ^ pl_swz(r);
    const unsigned group_byte = tiles_byte + (unsigned)(slot * PL_STAGE * 2 + wave * 1024);
    pl_issue_panels<0>(kbase + row * row_bytes + 16 * chunk, group_byte);
    pl_issue_panels<0>(vbase + row * row_bytes + 16 * chunk, group_byte + PL_IMG * 2);
  };
#define PL_WAITCNT(n) __builtin_amdgcn_s_waitcnt(0x0F70 | ((n) & 15) | (((n) >> 4) << 14))

  issue_step(0, 0);
  issue_step(1, 1);

  // Query rows as the B operand: lane (c, g) holds Q[row][32 j + 8 g .. +8]; padded rows are 0.
  elem8 qf[2][PL_KJ];
#pragma unroll
  for (int rt = 0; rt < 2; ++rt) {
    const elem_t* row = CL_ARG_Q + ((i64)tok[rt] * CL_Q_HEADS + qhead[rt]) * CL_HEAD_DIM + 8 * g;
#pragma unroll
    for (int j = 0; j < PL_KJ; ++j) {
      u32x4 raw = ld16(row + 32 * j);
      if (!live[rt]) raw = (u32x4){0u, 0u, 0u, 0u};
      qf[rt][j] = as_elem8(raw);
    }
  }

  float m_run[2] = {CL_NEG_BIG, CL_NEG_BIG};   // running max of the scaled scores (log2 domain), uniform over g
  float l_run[2] = {0.f, 0.f};                 // this lane's share of the sum of the rounded weights (normalises out)
  float l_exact[2] = {0.f, 0.f};               // ... of the unrounded ones (the lse)
  f32x4 acc[2][PL_FB];                         // acc[rt][fb][r] = O[row][16 fb + 4 g + r]
#pragma unroll
  for (int rt = 0; rt < 2; ++rt)
#pragma unroll
    for (int fb = 0; fb < PL_FB; ++fb) acc[rt][fb] = (f32x4){0.f, 0.f, 0.f, 0.f};

  // this lane's operand offsets inside an image (elements)
  const int a_lo = c * 64 + ((g ^ pl_swz(c)) << 3);
  const int vtok = 4 * g + (c >> 2);
  const int v_lo = vtok * 64 + (((((c & 3) >> 1)) ^ pl_swz(vtok)) << 3) + 4 * (c & 1);

  for (int step = 0; step < n_steps; ++step) {
    // step's images: this wave's share has landed when at most the next step's loads are
    // outstanding; the barrier makes that everybody's share and frees the images of step - 1
    PL_WAITCNT(PL_UNITS_PER);
    __syncthreads();
#if !CL_RAGGED
    // the loads enter a new window: its entries were read a window ago; read the one after it now
    const bool new_window = (step + 2) % (PL_WINDOW / PL_STEP) == 0 && step + 2 < n_steps;
    if (new_window) {
#pragma unroll
      for (int k = 0; k < 4; ++k) ids_cur[k] = ids_next[k];
    }
#endif
    issue_step(step + 2, (step + 2) % PL_STAGES);
#if !CL_RAGGED
    if (new_window) load_window((step + 2) / (PL_WINDOW / PL_STEP) + 1, ids_next);
#endif
    const elem_t* kimg = pl_tiles + (step % PL_STAGES) * PL_STAGE;
    const elem_t* vimg = kimg + PL_IMG;
    const int t0 = step * PL_STEP;

    // scores^T for the two 16-key halves and the wave's two row tiles
    f32x4 st[2][2];
#pragma unroll
    for (int rt = 0; rt < 2; ++rt) st[rt][0] = st[rt][1] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < PL_KJ; ++j)
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const elem8 a = *reinterpret_cast<const elem8*>(kimg + (j >> 1) * PL_PANEL + 16 * h * 64 +
                                                        (a_lo ^ ((4 * (j & 1)) << 3)));
#pragma unroll
        for (int rt = 0; rt < 2; ++rt) st[rt][h] = mfma16(a, qf[rt][j], st[rt][h]);
      }

    elem8 pf[2];
#pragma unroll
    for (int rt = 0; rt < 2; ++rt) {
      float s[8];
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int t = t0 + 16 * h + 4 * g + q;
          s[4 * h + q] = (t < ext && t <= limit[rt]) ? st[rt][h][q] * scale2 : CL_NEG_BIG;
        }
      float mx = s[0];
#pragma unroll
      for (int i = 1; i < 8; ++i) mx = fmaxf(mx, s[i]);
      mx = fmaxf(mx, lane_xor(mx, lane, 16));
      mx = fmaxf(mx, lane_xor(mx, lane, 32));
      const float m_new = fmaxf(m_run[rt], mx);
      const float alpha = fast_exp2(m_run[rt] - m_new);
      m_run[rt] = m_new;
      float psum = 0.f, esum = 0.f;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        // masked slots hold CL_NEG_BIG; when the whole row is still masked m_new equals it too,
        // so test the mask itself rather than trusting exp2 of a zero difference
        const float p = s[i] > 0.5f * CL_NEG_BIG ? fast_exp2(s[i] - m_new) : 0.f;
        const elem_t pe = to_elem(p);
        psum += to_f32(pe);
        esum += p;
        pf[rt][i] = pe;
      }
      l_run[rt] = l_run[rt] * alpha + psum;
      l_exact[rt] = l_exact[rt] * alpha + esum;
      if (__builtin_amdgcn_ballot_w64(alpha != 1.0f)) {   // wave-uniform: skip when no max moved
#pragma unroll
        for (int fb = 0; fb < PL_FB; ++fb) acc[rt][fb] *= alpha;
      }
    }

    // out^T block fb: rows = features 16 fb + (0..15), slots = keys 4 g + (0..3), 16 + 4 g + (0..3)
#pragma unroll
    for (int fb = 0; fb < PL_FB; ++fb) {
      const elem_t* p = vimg + (fb >> 2) * PL_PANEL + (v_lo ^ (((2 * fb) & 7) << 3));
      const pl_s16x4 lo4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((pl_lds_s16x4*)(p));
      const pl_s16x4 hi4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((pl_lds_s16x4*)(p + 16 * 64));
      const elem8 a = __builtin_bit_cast(elem8, (pl_s16x8)__builtin_shufflevector(lo4, hi4, 0, 1, 2, 3, 4, 5, 6, 7));
#pragma unroll
      for (int rt = 0; rt < 2; ++rt) acc[rt][fb] = mfma16(a, pf[rt], acc[rt][fb]);
    }
  }
  // no load may still be on its way into LDS when the workgroup ends
  PL_WAITCNT(0);

  // ---- each lane writes its rows' features (a row that saw no key: 0 and lse -inf) --------------
#pragma unroll
  for (int rt = 0; rt < 2; ++rt) {
    float l = l_run[rt], le = l_exact[rt];
    l += lane_xor(l, lane, 16);
    l += lane_xor(l, lane, 32);
    le += lane_xor(le, lane, 16);
    le += lane_xor(le, lane, 32);
    if (!live[rt]) continue;
    const float inv = 1.0f / fmaxf(l, 1.0e-30f);
    const i64 orow = (i64)tok[rt] * CL_Q_HEADS + qhead[rt];
    elem_t* dst = CL_ARG_OUT + orow * CL_HEAD_DIM + 4 * g;
#pragma unroll
    for (int fb = 0; fb < PL_FB; ++fb) {
      elem4 y;
#pragma unroll
      for (int r = 0; r < 4; ++r) y[r] = to_elem(acc[rt][fb][r] * inv);
      *reinterpret_cast<elem4*>(dst + 16 * fb) = y;
    }
#if CL_EMIT_LSE
    if (g == 0) CL_ARG_LSE[orow] = le > 0.f ? m_run[rt] + fast_log2(le) : CL_NEG_INF;
#endif
  }
}
#endif  // CL_EMIT_PARTIAL
