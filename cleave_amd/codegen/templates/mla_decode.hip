// ---- MLA decode: out = softmax((q kv^T + q_pe k_pe^T) * scale) kv, latent kv shared by heads --
//
// One workgroup owns (batch entry, 16*HG*WAVES heads, KV split).  A 32-token step of the latent
// (CL_CKV wide) and rope (CL_KPE wide) rows goes from global memory straight into LDS
// (global_load_lds, 16 bytes per lane: no staging registers, no LDS store instructions) as one
// token-major image shared by every wave:
//   tile  [D/64][32][64]   64-feature panels with 128-byte token rows; the 16-byte chunk index of
//                          a row is XORed with (token & 6)
// The score product (contraction over features) reads its A operand with one 16-byte LDS read
// per fragment; the value product (contraction over tokens) reads the same image with
// transposing reads (ds_read_b64_tr_b16: lane c of sixteen receives four consecutive tokens of
// feature c), so no feature-major copy exists.  Both read shapes are free of bank conflicts with
// that XOR.  CL_STAGES images rotate: while one is in the matrix cores the loads of the next
// CL_STAGES - 1 steps are in flight.
//
// Each wave owns 16*HG heads end to end and uses every operand it reads from LDS for HG matrix
// ops (LDS -> register bandwidth, about 32 bytes per clock and SIMD, is what bounds this kernel).
// scores^T = tile * Q^T with the Q fragments resident in registers, exact softmax lane-locally
// against a fixed reference point, then out^T += tile^T * P^T with P^T taken from the score
// registers in place.  Nothing is exchanged between waves; one barrier per step.
//
// The softmax reference point of a head is only raised when a score exceeds it by more than 8 (a
// factor 256): softmax is invariant to the reference point, weights stay below 2^8 and the
// accumulators are rescaled a handful of times per split, outside the hot loop.
//
//   CL_HEADS  heads per batch entry                    CL_CKV  latent width (multiple of 64)
//   CL_KPE    rope width (multiple of 64)              CL_SKV  kv length
//   CL_WAVES  waves per workgroup (1, 2, 4 or 8)       CL_HG   16-head groups per wave (1 or 2)
//   CL_SPLITS KV splits                                CL_BATCH  batch entries
//   CL_SCALE_LOG2E  softmax scale * log2(e)            CL_STAGES LDS images (2..4)
//   CL_OCC     workgroups meant to share a compute unit (register cap)
//   CL_VSPLIT  waves sharing one head set, each accumulating 1 / VSPLIT of the value features (the
//              accumulators of 32 heads x 512 features would fill a whole register class)
//   CL_PO_ELEM  1: split partials are normalised values in the element type with m = log-sum-exp
//               and l = 1;  0: unnormalised f32 values with the running (m, l)

#ifndef CL_HG
#define CL_HG 1
#endif
#ifndef CL_PO_ELEM
#define CL_PO_ELEM 0
#endif
#ifndef CL_STAGES
#define CL_STAGES 3
#endif
#define ML_STEP 32
#define ML_D (CL_CKV + CL_KPE)
#define ML_THREADS (CL_WAVES * 64)
#define ML_PANEL (ML_STEP * 64)               // elements of one 64-feature panel of the tile
#define ML_PANELS (ML_D / 64)
#define ML_LAT_PANELS (CL_CKV / 64)
#define ML_TILE (ML_PANELS * ML_PANEL)        // elements of one LDS image
#define ML_KJ (ML_D / 32)                     // score MFMAs per 16 tokens and head group
#define ML_FB (CL_CKV / 16)                   // 16-feature blocks of the value product
#ifndef CL_VSPLIT
#define CL_VSPLIT 1
#endif
#define ML_FBW (ML_FB / CL_VSPLIT)            // value feature blocks one wave accumulates
#define ML_HEADS_PER_BLOCK (16 * CL_HG * CL_WAVES / CL_VSPLIT)
#define ML_HEAD_GROUPS (CL_HEADS / ML_HEADS_PER_BLOCK)
#define ML_UNITS (ML_PANELS * 4)              // 1 KiB wave loads per step: (panel, 8-token group)
#define ML_LOAD_WAVES (CL_WAVES < 4 ? CL_WAVES : 4)        // waves that issue loads (the first ones)
#define ML_UNITS_PER (ML_UNITS / ML_LOAD_WAVES)
#define ML_RG_PER (4 / ML_LOAD_WAVES)                     // 8-token groups a loading wave takes
#define ML_AHEAD (CL_STAGES - 1)              // steps of loads in flight
#define ML_RESCALE_STEP 8.0f
#ifndef CL_LDS_AHEAD
#define CL_LDS_AHEAD 8
#endif
#define ML_LDS_AHEAD CL_LDS_AHEAD             // LDS operand reads in flight ahead of the matrix cores
static_assert(CL_CKV % 64 == 0 && CL_KPE % 64 == 0, "latent and rope widths are whole 64-feature panels");
static_assert(CL_HEADS % ML_HEADS_PER_BLOCK == 0, "heads divide into workgroups");
static_assert(CL_WAVES % CL_VSPLIT == 0 && ML_FB % (4 * CL_VSPLIT) == 0, "value features split into whole panels per wave");
static_assert(CL_SCALE_LOG2E > 0.f, "the largest raw score must be the largest scaled one");
static_assert(CL_WAVES == 1 || CL_WAVES == 2 || CL_WAVES == 4 || CL_WAVES == 8,
              "a loading wave takes whole 8-token groups of every panel");
static_assert(CL_STAGES >= 2 && CL_STAGES <= 4 && (ML_AHEAD - 1) * ML_UNITS_PER < 64, "load counter range");
constexpr bool ML_RAGGED = CL_SKV % ML_STEP != 0;   // the last step has tokens past the end

__shared__ __attribute__((aligned(1024))) elem_t ml_tiles[CL_STAGES * ML_TILE];

typedef short ml_s16x4 __attribute__((ext_vector_type(4)));
typedef short ml_s16x8 __attribute__((ext_vector_type(8)));
typedef __attribute__((address_space(3))) ml_s16x4 ml_lds_s16x4;

// chunk XOR of a token row: conflict-free for the 16-byte operand reads (lane = row l % 16, chunk
// l / 16 [+ 4]) and for the transposing 8-byte reads (a half wave reads tokens 4 g + i, i < 4,
// of two lane groups g, two neighbouring chunks each)
CL_DEVICE int ml_swz(int token) { return token & 6; }

// 16 bytes per lane, global -> LDS: the wave's 64 lanes fill 1 KiB starting at LDS byte address
// `lds_byte` + OFF (wave-uniform), lane l from `gptr` + OFF (the instruction's offset applies to
// both sides).  The load is invisible to the compiler's wait-count bookkeeping: the kernel waits
// for it itself (it counts as one vector memory operation of the wave).
template <int OFF>
CL_DEVICE void ml_dma16(const void* gptr, unsigned lds_byte) {
  // (readfirstlane: the LDS address is uniform by construction, the operand must be scalar by type)
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off offset:%2"
               :: "v"(gptr), "s"(__builtin_amdgcn_readfirstlane(lds_byte)), "n"(OFF) : "memory", "m0");
}

// A loading wave (the first four at most) takes, of every panel, the 8-token groups
// rg = wave * RG_PER + (0 .. RG_PER-1) (one group with four waves).  Lane l of a load takes token row l / 8 of the group and the chunk
// that belongs in slot l % 8 of that row.
struct MlLoader {
  u32 lat_off[ML_RG_PER];   // byte offset of this lane's chunk from the step's first latent row, panel 0
  u32 pe_off[ML_RG_PER];    // the same in the rope rows
};

CL_DEVICE void ml_loader_init(MlLoader& ld, int wave) {
  const int lane = threadIdx.x & 63;
#pragma unroll
  for (int q = 0; q < ML_RG_PER; ++q) {
    const int r = 8 * (wave * ML_RG_PER + q) + (lane >> 3);
    const int chunk = (lane & 7) ^ ml_swz(r);
    ld.lat_off[q] = (u32)((r * CL_CKV + 8 * chunk) * 2);
    ld.pe_off[q] = (u32)((r * CL_KPE + 8 * chunk) * 2);
  }
}

// loads of panel P, group q of this wave, and on to the next
template <int P, int Q>
CL_DEVICE void ml_issue_from(const MlLoader& ld, const elem_t* lat_rows, const elem_t* pe_rows, int t0,
                             unsigned stage_byte, int wave) {
  if constexpr (P < ML_PANELS) {
    const int rg = wave * ML_RG_PER + Q;
    // LDS target of lane 0: panel P, token row 8 rg; the instruction offset is taken back out
    constexpr int OFF = 128 * (P < ML_LAT_PANELS ? P : P - ML_LAT_PANELS);
    const unsigned lds_byte = stage_byte + (unsigned)(P * ML_PANEL * 2 + rg * 1024);
    if (ML_RAGGED) {
      // tokens past the end are clamped onto the last one (their scores are masked later)
      const int lane = threadIdx.x & 63;
      const int r = 8 * rg + (lane >> 3);
      int t = t0 + r;
      t = t < CL_SKV - 1 ? t : CL_SKV - 1;
      const int chunk = (lane & 7) ^ ml_swz(r);
      const elem_t* src = P < ML_LAT_PANELS ? lat_rows + (i64)(t - t0) * CL_CKV + 64 * P + 8 * chunk
                                            : pe_rows + (i64)(t - t0) * CL_KPE + 64 * (P - ML_LAT_PANELS) + 8 * chunk;
      ml_dma16<0>(src, lds_byte);
    } else {
      const char* src = P < ML_LAT_PANELS ? reinterpret_cast<const char*>(lat_rows) + ld.lat_off[Q]
                                          : reinterpret_cast<const char*>(pe_rows) + ld.pe_off[Q];
      ml_dma16<OFF>(src, lds_byte - OFF);
    }
    if constexpr (Q + 1 < ML_RG_PER) ml_issue_from<P, Q + 1>(ld, lat_rows, pe_rows, t0, stage_byte, wave);
    else ml_issue_from<P + 1, 0>(ld, lat_rows, pe_rows, t0, stage_byte, wave);
  }
}

#if CL_EMIT_PARTIAL
#ifndef CL_OCC
#define CL_OCC 1
#endif
// CL_OCC workgroups share a compute unit (the second launch bound caps the registers so that
// CL_OCC * WAVES / 4 waves fit a SIMD): their barriers are independent, so one's waits overlap
// the other's matrix work
extern "C" __global__ void __launch_bounds__(ML_THREADS, (CL_OCC * CL_WAVES + 3) / 4)
CL_PARTIAL_NAME(CL_PARTIAL_PARAMS) {
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int c = lane & 15, g = lane >> 4;
  // Workgroups go to the eight XCDs (one L2 each) round-robin in launch order.  The head blocks
  // that read the same rows (one batch entry, one split) are given launch ids 8 apart, so they
  // run on one XCD at about the same time and all but the first find the rows in its L2.
  int b, split, hg_block;
  {
    constexpr int units = CL_BATCH * CL_SPLITS;            // (batch entry, split) pairs
    const int launch = blockIdx.y * gridDim.x + blockIdx.x;
    if (units % 8 == 0) {
      hg_block = (launch / 8) % ML_HEAD_GROUPS;
      const int unit = (launch % 8) + 8 * (launch / (8 * ML_HEAD_GROUPS));
      b = unit / CL_SPLITS;
      split = unit % CL_SPLITS;
    } else {
      split = blockIdx.y;
      b = blockIdx.x / ML_HEAD_GROUPS;
      hg_block = blockIdx.x % ML_HEAD_GROUPS;
    }
  }
  // CL_VSPLIT neighbouring waves share one set of 16 * HG heads: each computes the set's scores
  // and accumulates its own 1 / VSPLIT of the value features
  const int head_set = wave / CL_VSPLIT, vhalf = wave % CL_VSPLIT;
  const int head0 = (hg_block * (CL_WAVES / CL_VSPLIT) + head_set) * 16 * CL_HG;   // this wave's first head

  const elem_t* kv = CL_ARG_KV + (i64)b * CL_SKV * CL_CKV;
  const elem_t* kpe = CL_ARG_KPE + (i64)b * CL_SKV * CL_KPE;
  const i64 row0 = (i64)b * CL_HEADS + head0;            // flattened (batch, head) row of the first head

  constexpr int n_steps = (CL_SKV + ML_STEP - 1) / ML_STEP;
  constexpr int per_split = (n_steps + CL_SPLITS - 1) / CL_SPLITS;
  const int step_begin = split * per_split;
  int step_end = step_begin + per_split;
  step_end = step_end < n_steps ? step_end : n_steps;
  const unsigned tiles_byte = (unsigned)(size_t)(__attribute__((address_space(3))) elem_t*)ml_tiles;

  float m_run[CL_HG];                  // softmax reference point of head c (log2 domain), uniform over g
  f32x4 l_acc[CL_HG];                  // every component: sum of the weights of head c
  f32x4 acc[CL_HG][ML_FBW];            // acc[hg][fb][r] = O[head 16 hg + c][16 (vhalf * FBW + fb) + 4 g + r]
#pragma unroll
  for (int hg = 0; hg < CL_HG; ++hg) {
    m_run[hg] = CL_NEG_BIG;
    l_acc[hg] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int fb = 0; fb < ML_FBW; ++fb) acc[hg][fb] = (f32x4){0.f, 0.f, 0.f, 0.f};
  }
  elem8 ones;
#pragma unroll
  for (int i = 0; i < 8; ++i) ones[i] = to_elem(1.0f);

  MlLoader ld;
  ml_loader_init(ld, wave);
  // Loads are issued for every step index, clamped onto the split's last step: the counter then
  // holds ML_AHEAD steps at every wait, also at the end of the split (the clamped loads refill
  // an image nobody reads any more).
#define ML_ISSUE(s)                                                                                   \
  {                                                                                                   \
    int s_ = (s) < step_end - 1 ? (s) : step_end - 1;                                                 \
    s_ = s_ > step_begin ? s_ : step_begin;                                                           \
    const int t0_ = s_ * ML_STEP;                                                                     \
    if (CL_WAVES <= 4 || wave < 4)                                                                    \
      ml_issue_from<0, 0>(ld, kv + (i64)t0_ * CL_CKV, kpe + (i64)t0_ * CL_KPE, t0_,                   \
                          tiles_byte + (unsigned)((((s) - step_begin) % CL_STAGES) * ML_TILE * 2), wave); \
  }
  // The image of step s is ready when all but the loads of the ML_AHEAD - 1 younger steps have
  // landed (this wave's share) and every wave has passed the barrier (everybody's share; also:
  // everybody is done reading the image that the next loads overwrite).
#define ML_WAIT_N ((ML_AHEAD - 1) * ML_UNITS_PER)
#define ML_FRONT(s)                                                                                   \
  __builtin_amdgcn_s_waitcnt(0x0F70 | (ML_WAIT_N & 15) | ((ML_WAIT_N >> 4) << 14));                   \
  __syncthreads();                                                                                    \
  ML_ISSUE((s) + ML_AHEAD)

  // The first ML_AHEAD steps' tile loads go out first, the Q fragments right behind them, and one
  // wait covers both (their latencies overlap).  After it the wave's vector-memory counter only
  // ever counts tile loads, ML_UNITS_PER per step, and they land in issue order: waiting until at
  // most (ML_AHEAD - 1) steps' loads are outstanding means every older step has landed.
  if (step_begin < step_end) {
#pragma unroll
    for (int i = 0; i < ML_AHEAD; ++i) ML_ISSUE(step_begin + i)
  }
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

  __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0)
  if (step_begin < step_end) {
    __syncthreads();
    ML_ISSUE(step_begin + ML_AHEAD)
  }

  // this lane's operand offsets inside an image (elements):
  //   score operand: token row c of a 16-token half, chunk g of a 32-feature block
  //   value operand: its 8-byte piece of the 4 (token) x 16 (feature) patch of lane group g
  const int a_lo = c * 64 + ((g ^ ml_swz(c)) << 3);
  const int vtok = 4 * g + (c >> 2);
  const int v_lo = vhalf * (ML_FBW / 4) * ML_PANEL + vtok * 64 + (((((c & 3) >> 1)) ^ ml_swz(vtok)) << 3) + 4 * (c & 1);

  // The hot loop runs with a fixed softmax reference point per head: weights are
  // exp2(score - m_run), their row sums come from one more matrix op against a tile of ones (the
  // sum then uses exactly the rounded weights the value product sees), and nothing crosses
  // lanes.  A lane whose scores exceed the reference by more than ML_RESCALE_STEP makes the
  // wave leave the loop before consuming the step; the cold block below raises the reference,
  // rescales (l, O) and re-enters at the same step (its scores are recomputed; the step's image
  // stays valid until the wave passes the next barrier).  Keeping the rescale outside the loop
  // keeps the accumulators where the matrix cores left them.
  int step = step_begin;
  for (;;) {
    bool raise_any = false;
    float mxl[CL_HG];                  // this lane's largest scaled score of the step that left the loop
    while (step < step_end) {
      const elem_t* tile = ml_tiles + ((step - step_begin) % CL_STAGES) * ML_TILE;

      // scores^T: rows = tokens 16 h + (0..15), columns = heads
      f32x4 st[CL_HG][2];
#pragma unroll
      for (int hg = 0; hg < CL_HG; ++hg) st[hg][0] = st[hg][1] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int j = 0; j < ML_KJ; ++j) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const elem8 a = *reinterpret_cast<const elem8*>(tile + (j >> 1) * ML_PANEL + 16 * h * 64 +
                                                          (a_lo ^ ((4 * (j & 1)) << 3)));
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
      if (step == step_begin && m_run[0] < 0.5f * CL_NEG_BIG) {
        // first step (nothing accumulated yet): its own maximum is the reference
#pragma unroll
        for (int hg = 0; hg < CL_HG; ++hg) {
          float mx = mxl[hg];
          mx = fmaxf(mx, lane_xor(mx, lane, 16));
          mx = fmaxf(mx, lane_xor(mx, lane, 32));
          m_run[hg] = mx;
        }
      } else if (__builtin_amdgcn_ballot_w64(raise)) {   // wave-uniform
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

      // out^T block fb: rows = features 16 fb + (0..15), slots = tokens 4 g + (0..3), 16 + 4 g + (0..3)
#pragma unroll
      for (int hg = 0; hg < CL_HG; ++hg) l_acc[hg] = mfma16(ones, pf[hg], l_acc[hg]);
#pragma unroll
      for (int fb = 0; fb < ML_FBW; ++fb) {
        const elem_t* p = tile + (fb >> 2) * ML_PANEL + (v_lo ^ (((2 * fb) & 7) << 3));
        const ml_s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((ml_lds_s16x4*)(p));
        const ml_s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((ml_lds_s16x4*)(p + 16 * 64));
        const elem8 a = __builtin_bit_cast(elem8, (ml_s16x8)__builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
#pragma unroll
        for (int hg = 0; hg < CL_HG; ++hg) acc[hg][fb] = mfma16(a, pf[hg], acc[hg][fb]);
      }
      __builtin_amdgcn_sched_group_barrier(0x100, ML_LDS_AHEAD, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, CL_HG, 0);
#pragma unroll
      for (int n = 0; n < ML_FBW - ML_LDS_AHEAD / 2; ++n) {
        __builtin_amdgcn_sched_group_barrier(0x008, CL_HG, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
      }
      __builtin_amdgcn_sched_group_barrier(0x008, CL_HG * (ML_LDS_AHEAD / 2), 0);

      ++step;
      if (step < step_end) {
        ML_FRONT(step)
      }
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
      for (int fb = 0; fb < ML_FBW; ++fb) acc[hg][fb] *= alpha;
    }
  }
  // no load may still be on its way into LDS when the workgroup ends
  __builtin_amdgcn_s_waitcnt(0x0F70);

  // ---- write this wave's heads (no cross-wave merge needed: a wave owns its heads) -------------
#pragma unroll
  for (int hg = 0; hg < CL_HG; ++hg) {
    const float l = l_acc[hg][0];
    const float m = m_run[hg];
    const i64 orow = row0 + 16 * hg + c;
    const int f0 = 16 * vhalf * ML_FBW + 4 * g;          // this lane's first feature of block 0
#if CL_SPLITS > 1 && !CL_PO_ELEM
    const i64 prow = (i64)split * CL_TOTAL_ROWS + orow;
#pragma unroll
    for (int fb = 0; fb < ML_FBW; ++fb)
      *reinterpret_cast<f32x4*>(CL_ARG_PO + prow * CL_CKV + f0 + 16 * fb) = acc[hg][fb];
    if (g == 0 && vhalf == 0) {
      CL_ARG_PM[prow] = m;
      CL_ARG_PL[prow] = l;
    }
#else
    const float inv = 1.0f / fmaxf(l, 1.0e-30f);
#if CL_SPLITS > 1
    const i64 prow = (i64)split * CL_TOTAL_ROWS + orow;
    elem_t* dst_row = CL_ARG_PO + prow * CL_CKV;
    if (g == 0 && vhalf == 0) {
      CL_ARG_PM[prow] = l > 0.f ? m + fast_log2(l) : CL_NEG_BIG;
      CL_ARG_PL[prow] = l > 0.f ? 1.0f : 0.f;
    }
#else
    elem_t* dst_row = CL_ARG_OUT + orow * CL_CKV;
#if CL_EMIT_LSE
    if (g == 0 && vhalf == 0) CL_ARG_LSE[orow] = l > 0.f ? m + fast_log2(l) : CL_NEG_INF;
#endif
#endif
#pragma unroll
    for (int fb = 0; fb < ML_FBW; ++fb) {
      elem4 y;
#pragma unroll
      for (int r = 0; r < 4; ++r) y[r] = to_elem(acc[hg][fb][r] * inv);
      *reinterpret_cast<elem4*>(dst_row + f0 + 16 * fb) = y;
    }
#endif
  }
}
#endif  // CL_EMIT_PARTIAL
