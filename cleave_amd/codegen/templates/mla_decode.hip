// ---- MLA decode: out = softmax((q kv^T + q_pe k_pe^T) * scale) kv, latent kv shared by heads --
//
// One workgroup owns (batch entry, 16*WAVES heads, KV split).  A 32-token step of the latent
// (CL_CKV wide) and rope (CL_KPE wide) rows is staged in LDS once and shared by every wave:
//   tile  [32][CKV + KPE]  token-major, for the score product (contraction over features)
//   vt    [CKV][32]        feature-major copy of the latent part, transposed 8x8 in registers
//                          on the way in, for the value product (contraction over tokens)
// Each wave owns 16 heads end to end: scores^T = tile * Q^T with its Q fragments resident in
// registers, exact online softmax lane-locally, then out^T += vt * P^T with P^T taken from
// the score registers in place (vt stores tokens in the slot order of that operand).  Nothing
// is exchanged between waves until the final merge; there is one barrier per step and the
// next step's global loads overlap the current step's matrix work.
//
//   CL_HEADS  heads per batch entry (multiple of 16)   CL_CKV  latent width (multiple of 32)
//   CL_KPE    rope width (multiple of 32)              CL_SKV  kv length
//   CL_WAVES  waves (= 16-head groups) per workgroup   CL_SPLITS  KV splits
//   CL_BATCH  batch entries                            CL_SCALE_LOG2E  softmax scale * log2(e)

#define ML_STEP 32
#define ML_D (CL_CKV + CL_KPE)
#define ML_THREADS (CL_WAVES * 64)
#define ML_TILE_LD (ML_D + 8)                 // token row pitch (elements)
#define ML_VT_LD (ML_STEP + 8)                // feature row pitch (elements)
#define ML_KJ (ML_D / 32)                     // score MFMAs per 16 tokens
#define ML_DT (CL_CKV / 16)                   // value MFMAs per step
#define ML_HEAD_GROUPS (CL_HEADS / (16 * CL_WAVES))
#define ML_LAT_BLOCKS (4 * (CL_CKV / 8))      // 8x8 latent blocks per step
#define ML_LAT_PER ((ML_LAT_BLOCKS + ML_THREADS - 1) / ML_THREADS)
#define ML_PE_CHUNKS (ML_STEP * (CL_KPE / 8)) // 16-byte rope chunks per step
#define ML_PE_PER ((ML_PE_CHUNKS + ML_THREADS - 1) / ML_THREADS)

struct MlStage {
  u32x4 lat[ML_LAT_PER][8];
  u32x4 pe[ML_PE_PER];
};

// token held by slot e of lane group g in the value product's contraction
CL_DEVICE int ml_slot_token(int g, int e) { return e < 4 ? 4 * g + e : 16 + 4 * g + (e - 4); }

CL_DEVICE void ml_load(const elem_t* __restrict__ kv, const elem_t* __restrict__ kpe, int t0, int kv_len,
                       MlStage& st) {
  const int last = kv_len - 1;
#pragma unroll
  for (int i = 0; i < ML_LAT_PER; ++i) {
    const int q = threadIdx.x + i * ML_THREADS;
    if (ML_LAT_BLOCKS % ML_THREADS == 0 || q < ML_LAT_BLOCKS) {
      const int db = q % (CL_CKV / 8), g = q / (CL_CKV / 8);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        int t = t0 + ml_slot_token(g, e);
        t = t < last ? t : last;
        st.lat[i][e] = ld16(kv + (i64)t * CL_CKV + 8 * db);
      }
    }
  }
#pragma unroll
  for (int i = 0; i < ML_PE_PER; ++i) {
    const int q = threadIdx.x + i * ML_THREADS;
    if (ML_PE_CHUNKS % ML_THREADS == 0 || q < ML_PE_CHUNKS) {
      int t = t0 + q / (CL_KPE / 8);
      t = t < last ? t : last;
      st.pe[i] = ld16(kpe + (i64)t * CL_KPE + 8 * (q % (CL_KPE / 8)));
    }
  }
}

CL_DEVICE void ml_store(const MlStage& st, elem_t* tile, elem_t* vt) {
#pragma unroll
  for (int i = 0; i < ML_LAT_PER; ++i) {
    const int q = threadIdx.x + i * ML_THREADS;
    if (ML_LAT_BLOCKS % ML_THREADS == 0 || q < ML_LAT_BLOCKS) {
      const int db = q % (CL_CKV / 8), g = q / (CL_CKV / 8);
#pragma unroll
      for (int e = 0; e < 8; ++e)
        *reinterpret_cast<u32x4*>(tile + ml_slot_token(g, e) * ML_TILE_LD + 8 * db) = st.lat[i][e];
      u32x4 t[8];
      transpose8x8(st.lat[i], t);
#pragma unroll
      for (int j = 0; j < 8; ++j) *reinterpret_cast<u32x4*>(vt + (8 * db + j) * ML_VT_LD + 8 * g) = t[j];
    }
  }
#pragma unroll
  for (int i = 0; i < ML_PE_PER; ++i) {
    const int q = threadIdx.x + i * ML_THREADS;
    if (ML_PE_CHUNKS % ML_THREADS == 0 || q < ML_PE_CHUNKS)
      *reinterpret_cast<u32x4*>(tile + (q / (CL_KPE / 8)) * ML_TILE_LD + CL_CKV + 8 * (q % (CL_KPE / 8))) = st.pe[i];
  }
}

#if CL_EMIT_PARTIAL
extern "C" __global__ void __launch_bounds__(ML_THREADS)
CL_PARTIAL_NAME(CL_PARTIAL_PARAMS) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int c = lane & 15, g = lane >> 4;
  const int split = blockIdx.y;
  const int b = blockIdx.x / ML_HEAD_GROUPS, hg = blockIdx.x % ML_HEAD_GROUPS;
  const int head0 = (hg * CL_WAVES + wave) * 16;         // this wave's first head

  const elem_t* kv = CL_ARG_KV + (i64)b * CL_SKV * CL_CKV;
  const elem_t* kpe = CL_ARG_KPE + (i64)b * CL_SKV * CL_KPE;
  const i64 row0 = (i64)b * CL_HEADS + head0;            // flattened (batch, head) row of head c = row0 + c

  constexpr int n_steps = (CL_SKV + ML_STEP - 1) / ML_STEP;
  constexpr int per_split = (n_steps + CL_SPLITS - 1) / CL_SPLITS;
  const int step_begin = split * per_split;
  int step_end = step_begin + per_split;
  step_end = step_end < n_steps ? step_end : n_steps;

  extern __shared__ __attribute__((aligned(16))) unsigned char ml_lds_raw[];
  elem_t* lds = reinterpret_cast<elem_t*>(ml_lds_raw);
  constexpr int TILE = ML_STEP * ML_TILE_LD, VT = CL_CKV * ML_VT_LD;
  elem_t* tiles = lds;                 // [2][32][TILE_LD]
  elem_t* vts = lds + 2 * TILE;        // [2][CKV][VT_LD]

  // Q fragments (B operand of the score product): lane (c, g) holds q[head c][32 j + 8 g .. +8]
  elem8 qf[ML_KJ];
#pragma unroll
  for (int j = 0; j < ML_KJ; ++j) {
    const int col = 32 * j + 8 * g;
    const elem_t* src = col < CL_CKV ? CL_ARG_Q + (row0 + c) * CL_CKV + col
                                     : CL_ARG_QPE + (row0 + c) * CL_KPE + (col - CL_CKV);
    qf[j] = as_elem8(ld16(src));
  }

  float m_run = CL_NEG_BIG, l_run = 0.f;
  f32x4 acc[ML_DT];                     // acc[i][r] = O[head c][16 i + 4 g + r]
#pragma unroll
  for (int i = 0; i < ML_DT; ++i) acc[i] = (f32x4){0.f, 0.f, 0.f, 0.f};

  MlStage stage;
  if (step_begin < step_end) {
    ml_load(kv, kpe, step_begin * ML_STEP, CL_SKV, stage);
    ml_store(stage, tiles, vts);
  }
  __syncthreads();

  for (int step = step_begin; step < step_end; ++step) {
    const int cur = (step - step_begin) & 1;
    const bool more = step + 1 < step_end;
    if (more) ml_load(kv, kpe, (step + 1) * ML_STEP, CL_SKV, stage);
    const elem_t* tile = tiles + cur * TILE;
    const elem_t* vt = vts + cur * VT;
    const int t0 = step * ML_STEP;

    float s[8];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      f32x4 st = (f32x4){0.f, 0.f, 0.f, 0.f};
      const elem_t* arow = tile + (16 * h + c) * ML_TILE_LD + 8 * g;
#pragma unroll
      for (int j = 0; j < ML_KJ; ++j) st = mfma16(*reinterpret_cast<const elem8*>(arow + 32 * j), qf[j], st);
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int t = t0 + 16 * h + 4 * g + r;
        s[4 * h + r] = t < CL_SKV ? st[r] * CL_SCALE_LOG2E : CL_NEG_BIG;
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
    float psum = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      float p = s[i] > 0.5f * CL_NEG_BIG ? fast_exp2(s[i] - m_new) : 0.f;
      elem_t pe = to_elem(p);
      psum += to_f32(pe);
      pf[i] = pe;
    }
    l_run = l_run * alpha + psum;
    if (__builtin_amdgcn_ballot_w64(alpha != 1.0f)) {
#pragma unroll
      for (int i = 0; i < ML_DT; ++i) acc[i] *= alpha;
    }
    // out^T tile i: rows = features 16 i + (0..15), A operand = vt rows, slots = tokens
    const elem_t* vrow = vt + c * ML_VT_LD + 8 * g;
#pragma unroll
    for (int i = 0; i < ML_DT; ++i)
      acc[i] = mfma16(*reinterpret_cast<const elem8*>(vrow + 16 * i * ML_VT_LD), pf, acc[i]);

    if (more) ml_store(stage, tiles + (cur ^ 1) * TILE, vts + (cur ^ 1) * VT);
    __syncthreads();
  }

  // ---- write this wave's heads (no cross-wave merge needed: a wave owns its heads) -------------
  l_run += lane_xor(l_run, lane, 16);
  l_run += lane_xor(l_run, lane, 32);
  const i64 orow = row0 + c;
#if CL_SPLITS > 1
  const i64 prow = (i64)split * CL_TOTAL_ROWS + orow;
#pragma unroll
  for (int i = 0; i < ML_DT; ++i) *reinterpret_cast<f32x4*>(CL_ARG_PO + prow * CL_CKV + 16 * i + 4 * g) = acc[i];
  if (g == 0) {
    CL_ARG_PM[prow] = m_run;
    CL_ARG_PL[prow] = l_run;
  }
#else
  const float inv = 1.0f / fmaxf(l_run, 1.0e-30f);
#pragma unroll
  for (int i = 0; i < ML_DT; ++i) {
    elem4 y;
#pragma unroll
    for (int r = 0; r < 4; ++r) y[r] = to_elem(acc[i][r] * inv);
    *reinterpret_cast<elem4*>(CL_ARG_OUT + orow * CL_CKV + 16 * i + 4 * g) = y;
  }
#if CL_EMIT_LSE
  if (g == 0) CL_ARG_LSE[orow] = l_run > 0.f ? m_run + fast_log2(l_run) : CL_NEG_INF;
#endif
#endif
}
#endif  // CL_EMIT_PARTIAL

