// ---- MLA decode: out = softmax((q kv^T + q_pe k_pe^T) * scale) kv, latent kv shared by heads --
//
// One workgroup owns (batch entry, 16*HG*WAVES heads, KV split).  A 32-token step of the latent
// (CL_CKV wide) and rope (CL_KPE wide) rows is staged in LDS once and shared by every wave:
//   tile  [D/64][32][64]   token-major in 64-feature panels (128-byte rows), for the score
//                          product (contraction over features)
//   vt    [CKV/2][64]      feature-major copy of the latent part (two features of 32 tokens per
//                          128-byte row), transposed 8x8 in registers on the way in, for the value
//                          product (contraction over tokens)
// Both use 128-byte rows with the 16-byte chunk index XORed by a function of the row, which makes
// the matrix-core operand reads and the staging writes free of bank conflicts (see ml_swz_*).
// Each wave owns 16*HG heads end to end and uses every operand it reads from LDS for HG matrix
// ops: with HG = 2 the LDS read traffic per flop is half that of one 16-head group per wave,
// which is what bounds this kernel.  scores^T = tile * Q^T with the Q fragments resident in
// registers, exact online softmax lane-locally, then out^T += vt * P^T with P^T taken from the
// score registers in place (vt stores tokens in the slot order of that operand).  Nothing is
// exchanged between waves; there is one barrier per step and the next step's global loads
// overlap the current step's matrix work.
//
// The softmax reference point of a head is only raised when a score exceeds it by more than 8 (a
// factor 256): softmax is invariant to the reference point, weights stay below 2^8 and the
// accumulators are rescaled a handful of times per split, outside the hot loop.
//
//   CL_HEADS  heads per batch entry                    CL_CKV  latent width (multiple of 64)
//   CL_KPE    rope width (multiple of 64)              CL_SKV  kv length
//   CL_WAVES  waves per workgroup                      CL_HG   16-head groups per wave (1 or 2)
//   CL_SPLITS KV splits                                CL_BATCH  batch entries
//   CL_SCALE_LOG2E  softmax scale * log2(e)
//   CL_PO_ELEM  1: split partials are normalised values in the element type with m = log-sum-exp
//               and l = 1;  0: unnormalised f32 values with the running (m, l)

#ifndef CL_HG
#define CL_HG 1
#endif
#ifndef CL_PO_ELEM
#define CL_PO_ELEM 0
#endif
#define ML_STEP 32
#define ML_D (CL_CKV + CL_KPE)
#define ML_THREADS (CL_WAVES * 64)
#define ML_PANEL (ML_STEP * 64)               // elements of one 64-feature panel of the tile
#define ML_KJ (ML_D / 32)                     // score MFMAs per 16 tokens and head group
#define ML_VI (CL_CKV / 32)                   // 16-row blocks of vt (each row holds two features)
#define ML_HEADS_PER_BLOCK (16 * CL_HG * CL_WAVES)
#define ML_HEAD_GROUPS (CL_HEADS / ML_HEADS_PER_BLOCK)
#define ML_LAT_BLOCKS (4 * (CL_CKV / 8))      // 8x8 latent blocks per step
#define ML_LAT_PER ((ML_LAT_BLOCKS + ML_THREADS - 1) / ML_THREADS)
#define ML_PE_CHUNKS (ML_STEP * (CL_KPE / 8)) // 16-byte rope chunks per step
#define ML_PE_PER ((ML_PE_CHUNKS + ML_THREADS - 1) / ML_THREADS)
#define ML_RESCALE_STEP 8.0f
#ifndef CL_LDS_AHEAD
#define CL_LDS_AHEAD 8
#endif
#define ML_LDS_AHEAD CL_LDS_AHEAD             // LDS operand reads in flight ahead of the matrix cores
static_assert(CL_CKV % 64 == 0 && CL_KPE % 64 == 0, "latent and rope widths are whole 64-feature panels");
static_assert(CL_HEADS % ML_HEADS_PER_BLOCK == 0, "heads divide into workgroups");
static_assert(CL_SCALE_LOG2E > 0.f, "the largest raw score must be the largest scaled one");

// Chunk swizzles of the two LDS images.  A 16-byte-per-lane LDS read is served 16 lanes at a
// time ({0-3,12-15,20-23,24-27}, {4-11,16-19,28-31}, and the same in the upper half) over 256
// bytes of banks; a 16-byte write 8 consecutive lanes at a time over 128 bytes.  With 128-byte
// rows both functions make the operand read (lane = row l % 16, chunk l / 16 [+ 4]) conflict
// free; the tile's also covers writes of one row by 8 lanes, vt's writes of one chunk of rows
// r, r + 4, ..., r + 28 by 8 lanes (the rows eight neighbouring 8x8 blocks transpose into).
CL_DEVICE int ml_swz_tile(int row) { return ((row >> 1) ^ (row >> 3)) & 7; }
CL_DEVICE int ml_swz_vt(int row) { return ((row >> 1) ^ (row >> 2)) & 7; }
CL_DEVICE int ml_tile_off(int token, int chunk) {   // chunk: 16-byte chunk of the D-wide row
  return (chunk >> 3) * ML_PANEL + token * 64 + ((((chunk & 7)) ^ ml_swz_tile(token)) << 3);
}
CL_DEVICE int ml_vt_off(int row, int chunk) { return row * 64 + ((chunk ^ ml_swz_vt(row)) << 3); }

struct MlStage {
  u32x4 lat[ML_LAT_PER][8];
  u32x4 pe[ML_PE_PER];
};

// token offset (within a 32-token step, relative to 4 g) of slot e of lane group g in the value
// product's contraction: slots 0-3 are tokens 4 g + (0..3), slots 4-7 tokens 16 + 4 g + (0..3)
constexpr int ml_slot_row(int e) { return e < 4 ? e : 12 + e; }
constexpr bool ML_RAGGED = CL_SKV % ML_STEP != 0;   // the last step has tokens past the end

// What a thread needs to move its share of a step: byte offsets into the step's slab of global
// rows and element offsets into one LDS stage.  Everything that depends on the lane is computed
// once; a step adds a uniform base and compile-time constants.
struct MlMover {
  u32 lat_g[ML_LAT_PER];    // bytes from the slab's first latent row to row 4 g, features 8 db
  u32 pe_g[ML_PE_PER];      // bytes from the slab's first rope row to this thread's chunk
  int tile_l[ML_LAT_PER];   // tile element offset of (token 4 g, chunk db)
  int vt_l[ML_LAT_PER];     // vt element offset of (row 4 db, chunk g)
  int pe_l[ML_PE_PER];      // tile element offset of this thread's rope chunk
};

CL_DEVICE void ml_mover_init(MlMover& mv) {
#pragma unroll
  for (int i = 0; i < ML_LAT_PER; ++i) {
    const int q = threadIdx.x + i * ML_THREADS;
    const int db = q % (CL_CKV / 8), g = (q / (CL_CKV / 8)) & 3;
    mv.lat_g[i] = (u32)((4 * g * CL_CKV + 8 * db) * 2);
    mv.tile_l[i] = ml_tile_off(4 * g, db);
    mv.vt_l[i] = ml_vt_off(4 * db, g);
  }
#pragma unroll
  for (int i = 0; i < ML_PE_PER; ++i) {
    const int q = threadIdx.x + i * ML_THREADS;
    const int t = (q / (CL_KPE / 8)) & (ML_STEP - 1), ch = q % (CL_KPE / 8);
    mv.pe_g[i] = (u32)((t * CL_KPE + 8 * ch) * 2);
    mv.pe_l[i] = ml_tile_off(t, CL_CKV / 8 + ch);
  }
}

CL_DEVICE u32x4 ml_ldg(const elem_t* base, u32 byte_off) {
  return *reinterpret_cast<const u32x4*>(reinterpret_cast<const char*>(base) + byte_off);
}

// Issue the loads of the step whose first token is t0 (kv, kpe: this batch entry's rows).
CL_DEVICE void ml_load(const elem_t* __restrict__ kv, const elem_t* __restrict__ kpe, int t0, const MlMover& mv,
                       MlStage& st) {
  if (!ML_RAGGED) {
    const elem_t* lat_rows = kv + (i64)t0 * CL_CKV;      // uniform: the loads take it as a scalar base
    const elem_t* pe_rows = kpe + (i64)t0 * CL_KPE;
#pragma unroll
    for (int i = 0; i < ML_LAT_PER; ++i)
      if (ML_LAT_BLOCKS % ML_THREADS == 0 || threadIdx.x + i * ML_THREADS < ML_LAT_BLOCKS) {
#pragma unroll
        for (int e = 0; e < 8; ++e) st.lat[i][e] = ml_ldg(lat_rows, mv.lat_g[i] + (u32)(ml_slot_row(e) * CL_CKV * 2));
      }
#pragma unroll
    for (int i = 0; i < ML_PE_PER; ++i)
      if (ML_PE_CHUNKS % ML_THREADS == 0 || threadIdx.x + i * ML_THREADS < ML_PE_CHUNKS)
        st.pe[i] = ml_ldg(pe_rows, mv.pe_g[i]);
  } else {
    // tokens past the end are clamped onto the last one (their scores are masked later)
    const int last = CL_SKV - 1;
#pragma unroll
    for (int i = 0; i < ML_LAT_PER; ++i) {
      const int q = threadIdx.x + i * ML_THREADS;
      if (ML_LAT_BLOCKS % ML_THREADS == 0 || q < ML_LAT_BLOCKS) {
        const int db = q % (CL_CKV / 8), g = q / (CL_CKV / 8);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          int t = t0 + 4 * g + ml_slot_row(e);
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
}

// Write a loaded step into the LDS stage at `tile` / `vt`.  Both swizzles are XOR-linear in the
// row bits, and a thread's rows differ from its first one only in bits its lane does not set, so
// every address is (lane offset ^ constant) + constant.
CL_DEVICE void ml_store(const MlStage& st, const MlMover& mv, elem_t* tile, elem_t* vt) {
#pragma unroll
  for (int i = 0; i < ML_LAT_PER; ++i) {
    if (ML_LAT_BLOCKS % ML_THREADS == 0 || threadIdx.x + i * ML_THREADS < ML_LAT_BLOCKS) {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int row = ml_slot_row(e);   // token 4 g + row: tile row offset and swizzle term of `row`
        *reinterpret_cast<u32x4*>(tile + ((mv.tile_l[i] ^ (ml_swz_tile(row) << 3)) + row * 64)) = st.lat[i][e];
      }
      u32x4 t[8];
      transpose8x8(st.lat[i], t);
      // feature 8 db + j -> vt row 4 db + j / 2, chunk (4 (j % 2)) ^ g
#pragma unroll
      for (int j = 0; j < 8; ++j)
        *reinterpret_cast<u32x4*>(vt + ((mv.vt_l[i] ^ (((4 * (j & 1)) ^ ml_swz_vt(j >> 1)) << 3)) + (j >> 1) * 64)) = t[j];
    }
  }
#pragma unroll
  for (int i = 0; i < ML_PE_PER; ++i)
    if (ML_PE_CHUNKS % ML_THREADS == 0 || threadIdx.x + i * ML_THREADS < ML_PE_CHUNKS)
      *reinterpret_cast<u32x4*>(tile + mv.pe_l[i]) = st.pe[i];
}

#ifdef CL_DBG_TIMING
// debugging aid: wave 0 of every workgroup leaves cycle-counter readings in its PL rows
#define ML_STAMP(k) if (threadIdx.x == 0) reinterpret_cast<unsigned*>(CL_ARG_PL)[(blockIdx.y * gridDim.x + blockIdx.x) * 32 + (k)] = (unsigned)__builtin_readcyclecounter();
#else
#define ML_STAMP(k)
#endif

#if CL_EMIT_PARTIAL
extern "C" __global__ void __launch_bounds__(ML_THREADS)
CL_PARTIAL_NAME(CL_PARTIAL_PARAMS) {
  ML_STAMP(0)
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int c = lane & 15, g = lane >> 4;
  const int split = blockIdx.y;
  const int b = blockIdx.x / ML_HEAD_GROUPS, hg_block = blockIdx.x % ML_HEAD_GROUPS;
  const int head0 = (hg_block * CL_WAVES + wave) * 16 * CL_HG;   // this wave's first head

  const elem_t* kv = CL_ARG_KV + (i64)b * CL_SKV * CL_CKV;
  const elem_t* kpe = CL_ARG_KPE + (i64)b * CL_SKV * CL_KPE;
  const i64 row0 = (i64)b * CL_HEADS + head0;            // flattened (batch, head) row of the first head

  constexpr int n_steps = (CL_SKV + ML_STEP - 1) / ML_STEP;
  constexpr int per_split = (n_steps + CL_SPLITS - 1) / CL_SPLITS;
  const int step_begin = split * per_split;
  int step_end = step_begin + per_split;
  step_end = step_end < n_steps ? step_end : n_steps;

  extern __shared__ __attribute__((aligned(16))) unsigned char ml_lds_raw[];
  elem_t* lds = reinterpret_cast<elem_t*>(ml_lds_raw);
  constexpr int TILE = (ML_D / 64) * ML_PANEL, VT = (CL_CKV / 2) * 64;
  elem_t* tiles = lds;                 // [2][D/64][32][64]
  elem_t* vts = lds + 2 * TILE;        // [2][CKV/2][64]

  // Q fragments (B operand of the score product): lane (c, g) holds q[head c][32 j + 8 g .. +8]
  elem8 qf[CL_HG][ML_KJ];
#pragma unroll
  for (int hg = 0; hg < CL_HG; ++hg)
#pragma unroll
    for (int j = 0; j < ML_KJ; ++j) {
      const int col = 32 * j + 8 * g;
      const i64 row = row0 + 16 * hg + c;
      const elem_t* src = col < CL_CKV ? CL_ARG_Q + row * CL_CKV + col : CL_ARG_QPE + row * CL_KPE + (col - CL_CKV);
      qf[hg][j] = as_elem8(ld16(src));
    }

  float m_run[CL_HG];                  // softmax reference point of head c (log2 domain), uniform over g
  f32x4 l_acc[CL_HG];                  // every component: sum of the weights of head c
  f32x4 acc[CL_HG][ML_VI][2];          // acc[hg][i][hf][r] = O[head 16 hg + c][32 i + 8 g + 2 r + hf]
#pragma unroll
  for (int hg = 0; hg < CL_HG; ++hg) {
    m_run[hg] = CL_NEG_BIG;
    l_acc[hg] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < ML_VI; ++i) acc[hg][i][0] = acc[hg][i][1] = (f32x4){0.f, 0.f, 0.f, 0.f};
  }
  elem8 ones;
#pragma unroll
  for (int i = 0; i < 8; ++i) ones[i] = to_elem(1.0f);

  MlMover mv;
  ml_mover_init(mv);
  MlStage stage;
  if (step_begin < step_end) {
    ml_load(kv, kpe, step_begin * ML_STEP, mv, stage);
    ml_store(stage, mv, tiles, vts);
  }
  // every load issued so far (the Q fragments among them) has landed before the loop: a wait
  // inside the loop then never counts loads older than that step's own prefetch
  __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0)
  __syncthreads();
  ML_STAMP(1)

  // this lane's operand chunk offsets: row c of a 16-row block, chunk g
  const int a_lo = c * 64 + ((g ^ ml_swz_tile(c)) << 3);
  const int v_lo = c * 64 + ((g ^ ml_swz_vt(c)) << 3);

  // The hot loop runs with a fixed softmax reference point per head: weights are
  // exp2(score - m_run), their row sums come from one more matrix op against a tile of ones (the
  // sum then uses exactly the rounded weights the value product sees), and nothing crosses
  // lanes.  A lane whose scores exceed the reference by more than ML_RESCALE_STEP makes the
  // wave leave the loop before consuming the step; the cold block below raises the reference,
  // rescales (l, O) and re-enters at the same step (its scores are recomputed; its barrier has
  // not been reached yet, so every wave still meets exactly one barrier per step).  The first
  // step always takes that path, with (l, O) still zero.  Keeping the rescale outside the loop
  // keeps the accumulators where the matrix cores left them: inside, the compiler copies all of
  // them out on every step.
  int step = step_begin;
  for (;;) {
    bool raise_any = false;
    float mxl[CL_HG];                  // this lane's largest scaled score of the step that left the loop
    while (step < step_end) {
      const int cur = (step - step_begin) & 1;
      const bool more = step + 1 < step_end;
#ifndef CL_DBG_NOLOAD
      if (more) ml_load(kv, kpe, (step + 1) * ML_STEP, mv, stage);
#endif
      const elem_t* tile = tiles + cur * TILE;
      const elem_t* vt = vts + cur * VT;

      // scores^T: rows = tokens 16 h + (0..15), columns = heads
      f32x4 st[CL_HG][2];
#pragma unroll
      for (int hg = 0; hg < CL_HG; ++hg) st[hg][0] = st[hg][1] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int j = 0; j < ML_KJ; ++j) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          // row 16 h + c: swizzle(16 h + c) = swizzle(c) ^ (2 h)
          const elem8 a = *reinterpret_cast<const elem8*>(tile + (j >> 1) * ML_PANEL + 16 * h * 64 +
                                                          (a_lo ^ ((4 * (j & 1)) << 3) ^ ((2 * h) << 3)));
#pragma unroll
          for (int hg = 0; hg < CL_HG; ++hg) st[hg][h] = mfma16(a, qf[hg][j], st[hg][h]);
        }
      }
      // order of the above: the LDS operand reads stay ML_LDS_AHEAD ahead of the matrix ops that
      // consume them (one wave per SIMD: nothing else hides the LDS latency)
      __builtin_amdgcn_sched_group_barrier(0x100, ML_LDS_AHEAD, 0);
#pragma unroll
      for (int n = 0; n < 2 * ML_KJ - ML_LDS_AHEAD; ++n) {
        __builtin_amdgcn_sched_group_barrier(0x008, CL_HG, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      }
      __builtin_amdgcn_sched_group_barrier(0x008, CL_HG * ML_LDS_AHEAD, 0);

      if (ML_RAGGED) {
        const int t0 = step * ML_STEP;
#pragma unroll
        for (int hg = 0; hg < CL_HG; ++hg)
#pragma unroll
          for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int r = 0; r < 4; ++r)
              if (t0 + 16 * h + 4 * g + r >= CL_SKV) st[hg][h][r] = CL_NEG_BIG;   // weight exp2(-huge) = 0
      }
      bool raise = false;
#pragma unroll
      for (int hg = 0; hg < CL_HG; ++hg) {
        float v = fmaxf(fmaxf(st[hg][0][0], st[hg][0][1]), fmaxf(st[hg][0][2], st[hg][0][3]));
        v = fmaxf(v, fmaxf(fmaxf(st[hg][1][0], st[hg][1][1]), fmaxf(st[hg][1][2], st[hg][1][3])));
        mxl[hg] = v * CL_SCALE_LOG2E;
        raise = raise || mxl[hg] > m_run[hg] + ML_RESCALE_STEP;
      }
      if (__builtin_amdgcn_ballot_w64(raise)) {   // wave-uniform
        raise_any = true;
        break;
      }

      elem8 pf[CL_HG];
#pragma unroll
      for (int hg = 0; hg < CL_HG; ++hg)
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
          for (int r = 0; r < 4; ++r)
            pf[hg][4 * h + r] = to_elem(fast_exp2(__builtin_fmaf(st[hg][h][r], CL_SCALE_LOG2E, -m_run[hg])));

      // out^T block (i, hf): rows = vt rows 16 i + (0..15) = features 32 i + 2 row + hf, slots = tokens
#pragma unroll
      for (int hg = 0; hg < CL_HG; ++hg) l_acc[hg] = mfma16(ones, pf[hg], l_acc[hg]);
#pragma unroll
      for (int i = 0; i < ML_VI; ++i) {
#pragma unroll
        for (int hf = 0; hf < 2; ++hf) {
          // vt row 16 i + c: swizzle = swizzle(c) ^ (4 (i & 1))
          const elem8 a = *reinterpret_cast<const elem8*>(vt + 16 * i * 64 +
                                                          (v_lo ^ ((4 * hf) << 3) ^ ((4 * (i & 1)) << 3)));
#pragma unroll
          for (int hg = 0; hg < CL_HG; ++hg) acc[hg][i][hf] = mfma16(a, pf[hg], acc[hg][i][hf]);
        }
      }
      __builtin_amdgcn_sched_group_barrier(0x100, ML_LDS_AHEAD, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, CL_HG, 0);
#pragma unroll
      for (int n = 0; n < 2 * ML_VI - ML_LDS_AHEAD; ++n) {
        __builtin_amdgcn_sched_group_barrier(0x008, CL_HG, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      }
      __builtin_amdgcn_sched_group_barrier(0x008, CL_HG * ML_LDS_AHEAD, 0);

#ifndef CL_DBG_NOSTORE
      if (more) ml_store(stage, mv, tiles + (cur ^ 1) * TILE, vts + (cur ^ 1) * VT);
#endif
      __syncthreads();
      ++step;
      ML_STAMP(2 + (step - step_begin < 24 ? step - step_begin : 24))
    }
    if (!raise_any) break;
    // cold: raise the reference of the heads that need it and rescale what they have accumulated
#pragma unroll
    for (int hg = 0; hg < CL_HG; ++hg) {
      float mx = mxl[hg];
      mx = fmaxf(mx, lane_xor(mx, lane, 16));
      mx = fmaxf(mx, lane_xor(mx, lane, 32));
      const bool up = mx > m_run[hg] + ML_RESCALE_STEP;
      const float m_new = up ? mx : m_run[hg];
      const float alpha = up ? fast_exp2(m_run[hg] - m_new) : 1.0f;
      m_run[hg] = m_new;
      l_acc[hg] *= alpha;
#pragma unroll
      for (int i = 0; i < ML_VI; ++i) {
        acc[hg][i][0] *= alpha;
        acc[hg][i][1] *= alpha;
      }
    }
  }

  ML_STAMP(29)
  // ---- write this wave's heads (no cross-wave merge needed: a wave owns its heads) -------------
#pragma unroll
  for (int hg = 0; hg < CL_HG; ++hg) {
    const float l = l_acc[hg][0];
    const float m = m_run[hg];
    const i64 orow = row0 + 16 * hg + c;
#if CL_SPLITS > 1 && !CL_PO_ELEM
    const i64 prow = (i64)split * CL_TOTAL_ROWS + orow;
#pragma unroll
    for (int i = 0; i < ML_VI; ++i) {
      float* dst = CL_ARG_PO + prow * CL_CKV + 32 * i + 8 * g;
      *reinterpret_cast<f32x4*>(dst) = (f32x4){acc[hg][i][0][0], acc[hg][i][1][0], acc[hg][i][0][1], acc[hg][i][1][1]};
      *reinterpret_cast<f32x4*>(dst + 4) = (f32x4){acc[hg][i][0][2], acc[hg][i][1][2], acc[hg][i][0][3], acc[hg][i][1][3]};
    }
    if (g == 0) {
      CL_ARG_PM[prow] = m;
      CL_ARG_PL[prow] = l;
    }
#else
    const float inv = 1.0f / fmaxf(l, 1.0e-30f);
#if CL_SPLITS > 1
    const i64 prow = (i64)split * CL_TOTAL_ROWS + orow;
    elem_t* dst_row = CL_ARG_PO + prow * CL_CKV;
#ifndef CL_DBG_TIMING
    if (g == 0) {
      CL_ARG_PM[prow] = l > 0.f ? m + fast_log2(l) : CL_NEG_BIG;
      CL_ARG_PL[prow] = l > 0.f ? 1.0f : 0.f;
    }
#endif
#else
    elem_t* dst_row = CL_ARG_OUT + orow * CL_CKV;
#if CL_EMIT_LSE
    if (g == 0) CL_ARG_LSE[orow] = l > 0.f ? m + fast_log2(l) : CL_NEG_INF;
#endif
#endif
#pragma unroll
    for (int i = 0; i < ML_VI; ++i) {
      elem8 y;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        y[2 * r] = to_elem(acc[hg][i][0][r] * inv);
        y[2 * r + 1] = to_elem(acc[hg][i][1][r] * inv);
      }
      st16(dst_row + 32 * i + 8 * g, as_u32x4(y));
    }
#endif
  }
  ML_STAMP(30)
}
#endif  // CL_EMIT_PARTIAL
