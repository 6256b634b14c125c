// ---- MLA decode with score waves and value waves ------------------------------------------------
//
//   out = softmax((q kv^T + q_pe k_pe^T) * scale) kv        latent kv shared by all heads
//
// Same operator, operands, step size and LDS image as mla_decode.hip (a 32-token step of the
// latent and rope rows goes global -> LDS directly as one token-major image of 64-feature panels,
// 128-byte token rows, chunk index XOR (token & 6); score operands are 16-byte reads, value
// operands transposing reads of the same image).  What differs is who does what.  There, a wave
// owns 16 heads end to end, and every one of its 69 matrix ops per step is fed by a fresh 1 KiB
// LDS read: 272 KB out of LDS per step and 64 heads, at the ~128 bytes per clock a compute unit's
// LDS delivers twice as long as the matrix ops take.  Sharing an operand between two head tiles
// needs the registers of 32 heads (Q fragments 144, accumulators 256), which one wave does not
// have.  Two kinds of wave do:
//
//   score wave s (2 of them)    keeps the Q fragments of heads 32 s .. 32 s + 31; every key
//                               fragment it reads feeds two matrix ops (its two head tiles).  It
//                               makes the scores of step t, the softmax weights against its
//                               reference points, their row sums, and leaves the weights (as the
//                               value product's B operand, 16 bytes per lane and head tile) and a
//                               rescale factor per head in LDS;
//   value wave (s, f) (4)       keeps the accumulators of the same 32 heads for half of the
//                               latent features (2 x 16 x 16 x 16 values); every value fragment it
//                               reads feeds two matrix ops.  It picks the weights of step t - 1 up
//                               and adds their value product.  The value waves also issue every
//                               tile load.
//
// Per step and 64 heads that is 72 + 72 KB out of LDS for the same 276 matrix ops, which brings
// the two limits level.  The waves sit on the four SIMDs as {value, value}, {value, value},
// {score}, {score} (wave w runs on SIMD w % 4): 66 to 72 matrix ops per SIMD and step.  The loop is
// skewed by one step, one barrier per step: in iteration t the score waves read image t and the
// value waves image t - 1, the loads of images t + 1 and t + 2 are in flight (four images).
//
// Softmax reference: a head's reference point is raised only when a score passes it by 2^8; the
// score wave then also publishes alpha = 2^(old - new) for that step (1 otherwise) and the value
// waves multiply their accumulators by it before adding the step -- the factor travels with the
// weights it belongs to, so there is no handshake.  At the end the score waves hand over (m, l).
//
//   CL_HEADS (multiple of 64)  CL_CKV (multiple of 128)  CL_KPE (multiple of 64)  CL_SKV  CL_BATCH
//   CL_SPLITS  CL_SCALE_LOG2E  CL_PO_ELEM (1: split partials normalised, in the element type)

#ifndef CL_PO_ELEM
#define CL_PO_ELEM 0
#endif
#define MD_STEP 32
#define MD_D (CL_CKV + CL_KPE)
#define MD_PANEL (MD_STEP * 64)
#define MD_PANELS (MD_D / 64)
#define MD_LAT_PANELS (CL_CKV / 64)
#define MD_TILE (MD_PANELS * MD_PANEL)          // elements of one image
#define MD_STAGES 4
#define MD_KJ (MD_D / 32)
#define MD_FB (CL_CKV / 16)
#define MD_FBW (MD_FB / 2)                       // feature blocks one value wave accumulates
#define MD_THREADS 384
#define MD_HEADS_PER_BLOCK 64
#define MD_HEAD_GROUPS (CL_HEADS / MD_HEADS_PER_BLOCK)
#define MD_UNITS_PER MD_PANELS                  // 1 KiB loads per value wave and step: its 8-token group of every panel
#define MD_RESCALE_STEP 8.0f
#ifndef CL_LDS_AHEAD
#define CL_LDS_AHEAD 8
#endif
static_assert(CL_CKV % 128 == 0 && CL_KPE % 64 == 0, "whole 64-feature panels, the latent ones halved between two value waves");
static_assert(CL_HEADS % MD_HEADS_PER_BLOCK == 0, "64 heads per workgroup");
static_assert(CL_SCALE_LOG2E > 0.f, "the largest raw score must be the largest scaled one");
static_assert(MD_UNITS_PER < 32, "load counter range");
constexpr bool MD_RAGGED = CL_SKV % MD_STEP != 0;

__shared__ __attribute__((aligned(1024))) elem_t md_tiles[MD_STAGES * MD_TILE];
__shared__ __attribute__((aligned(16))) u32x4 md_weights[2][2][2][64]; // [step parity][head set][head tile][lane]: the lane's eight weights
__shared__ float md_alpha[2][2][2][64];                                // the same index: rescale factor of head lane % 16 of the tile
__shared__ float md_final[2][2][2][16];                                // [head set][head tile][m, l][head]

typedef short md_s16x4 __attribute__((ext_vector_type(4)));
typedef short md_s16x8 __attribute__((ext_vector_type(8)));
typedef __attribute__((address_space(3))) md_s16x4 md_lds_s16x4;

CL_DEVICE int md_swz(int token) { return token & 6; }

// 16 bytes per lane, global -> LDS; not counted by the compiler, the issuing wave waits itself
template <int OFF>
CL_DEVICE void md_dma16(const void* gptr, unsigned lds_byte) {
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off offset:%2"
               :: "v"(gptr), "s"(__builtin_amdgcn_readfirstlane(lds_byte)), "n"(OFF) : "memory", "m0");
}

// every LDS access of this wave has completed, then the workgroup barrier
CL_DEVICE void md_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// value wave `lw` (0..3): its loads of one step, panel P onwards -- token rows 8 lw + lane / 8 of
// every panel, the chunk that belongs in slot lane % 8
template <int P>
CL_DEVICE void md_issue_from(u32 lat_off, u32 pe_off, const elem_t* lat_rows, const elem_t* pe_rows, int t0,
                             unsigned stage_byte, int lw) {
  if constexpr (P < MD_PANELS) {
    constexpr int OFF = 128 * (P < MD_LAT_PANELS ? P : P - MD_LAT_PANELS);
    const unsigned lds_byte = stage_byte + (unsigned)(P * MD_PANEL * 2 + lw * 1024);
    if (MD_RAGGED) {
      // tokens past the end are clamped onto the last one (their scores are masked)
      const int lane = threadIdx.x & 63;
      const int r = 8 * lw + (lane >> 3);
      int t = t0 + r;
      t = t < CL_SKV - 1 ? t : CL_SKV - 1;
      const int chunk = (lane & 7) ^ md_swz(r);
      const elem_t* src = P < MD_LAT_PANELS ? lat_rows + (i64)(t - t0) * CL_CKV + 64 * P + 8 * chunk
                                            : pe_rows + (i64)(t - t0) * CL_KPE + 64 * (P - MD_LAT_PANELS) + 8 * chunk;
      md_dma16<0>(src, lds_byte);
    } else {
      const char* src = P < MD_LAT_PANELS ? reinterpret_cast<const char*>(lat_rows) + lat_off
                                          : reinterpret_cast<const char*>(pe_rows) + pe_off;
      md_dma16<OFF>(src, lds_byte - OFF);
    }
    md_issue_from<P + 1>(lat_off, pe_off, lat_rows, pe_rows, t0, stage_byte, lw);
  }
}

#if CL_EMIT_PARTIAL
extern "C" __global__ void __launch_bounds__(MD_THREADS)
CL_PARTIAL_NAME(CL_PARTIAL_PARAMS) {
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int c = lane & 15, g = lane >> 4;
  // waves 2, 3: score waves of head sets 0, 1; waves 0, 4 / 1, 5: value waves of head set 0 / 1,
  // feature halves 0, 1
  const bool scores = wave == 2 || wave == 3;
  const int set = scores ? wave - 2 : (wave & 1);
  const int fhalf = wave >> 2;
  const int loader = 2 * (wave & 1) + fhalf;              // value waves: which 8-token group of every panel they load
  // Workgroups go to the eight XCDs (one L2 each) round-robin in launch order.  Every workgroup
  // of a batch entry is given to one XCD (batch entry b to XCD b % 8): the head blocks of a split
  // read the same kv rows and the splits of a head block the same Q rows, so each row comes out of
  // HBM once and every other reader finds it in that L2.
  int b, split, hg_block;
  {
    constexpr int per_entry = CL_SPLITS * MD_HEAD_GROUPS;
    const int launch = blockIdx.y * gridDim.x + blockIdx.x;
    if (CL_BATCH % 8 == 0) {
      const int k = launch / 8;                              // the k-th workgroup of XCD launch % 8
      b = launch % 8 + 8 * (k / per_entry);
      split = (k % per_entry) / MD_HEAD_GROUPS;
      hg_block = k % MD_HEAD_GROUPS;
    } else {
      split = blockIdx.y;
      b = blockIdx.x / MD_HEAD_GROUPS;
      hg_block = blockIdx.x % MD_HEAD_GROUPS;
    }
  }
  const int head0 = hg_block * MD_HEADS_PER_BLOCK + 32 * set;      // first head of this wave's head set
  const elem_t* kv = CL_ARG_KV + (i64)b * CL_SKV * CL_CKV;
  const elem_t* kpe = CL_ARG_KPE + (i64)b * CL_SKV * CL_KPE;
  const i64 row0 = (i64)b * CL_HEADS + head0;

  constexpr int n_steps = (CL_SKV + MD_STEP - 1) / MD_STEP;
  constexpr int per_split = (n_steps + CL_SPLITS - 1) / CL_SPLITS;
  const int step_begin = split * per_split;
  int step_end = step_begin + per_split;
  step_end = step_end < n_steps ? step_end : n_steps;
  const int n_own = step_end > step_begin ? step_end - step_begin : 0;       // steps of this split
  const unsigned tiles_byte = (unsigned)(size_t)(__attribute__((address_space(3))) elem_t*)md_tiles;

  if (scores) {
    // =========================================================================== score wave
    // Q fragments (B operand): lane (c, g) holds q[head 16 t + c][32 j + 8 g .. + 8] for head tile t
    elem8 qf[2][MD_KJ];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int j = 0; j < MD_KJ; ++j) {
        const int col = 32 * j + 8 * g;
        const i64 row = row0 + 16 * t + c;
        const elem_t* src = col < CL_CKV ? CL_ARG_Q + row * CL_CKV + col : CL_ARG_QPE + row * CL_KPE + (col - CL_CKV);
        qf[t][j] = as_elem8(ld16(src));
      }
    elem8 ones;
#pragma unroll
    for (int i = 0; i < 8; ++i) ones[i] = to_elem(1.0f);
    float m_run[2] = {CL_NEG_BIG, CL_NEG_BIG};      // reference point of head c of each tile (log2 domain), uniform over g
    f32x4 l_acc[2];                                 // every component: sum of the weights of head c
    l_acc[0] = l_acc[1] = (f32x4){0.f, 0.f, 0.f, 0.f};
    const int a_lo = c * 64 + ((g ^ md_swz(c)) << 3);

    for (int it = 0; it <= n_own; ++it) {
      md_barrier();                                 // image `it` has landed (the value waves waited for it)
      if (it == n_own) break;
      const elem_t* tile = md_tiles + (it % MD_STAGES) * MD_TILE;
#ifdef CL_DBG_NOS
      continue;
#endif
      // scores^T: rows = tokens 16 h + (0..15), columns = heads of tile t
      f32x4 st[2][2];
#pragma unroll
      for (int t = 0; t < 2; ++t) st[t][0] = st[t][1] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int j = 0; j < MD_KJ; ++j)
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const elem8 a = *reinterpret_cast<const elem8*>(tile + (j >> 1) * MD_PANEL + 16 * h * 64 +
                                                          (a_lo ^ ((4 * (j & 1)) << 3)));
#pragma unroll
          for (int t = 0; t < 2; ++t) st[t][h] = mfma16(a, qf[t][j], st[t][h]);
        }
      // the operand reads stay CL_LDS_AHEAD ahead of the matrix ops that consume them.  (Working the
      // first token half's weights out between the second half's matrix ops was measured and is
      // no faster: a wave alone on its SIMD issues its vector and matrix instructions one after
      // the other either way.)
      __builtin_amdgcn_sched_group_barrier(0x100, CL_LDS_AHEAD, 0);
#pragma unroll
      for (int n = 0; n < 2 * MD_KJ - CL_LDS_AHEAD; ++n) {
        __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      }
      __builtin_amdgcn_sched_group_barrier(0x008, 2 * CL_LDS_AHEAD, 0);

      if (MD_RAGGED) {
        const int t0 = (step_begin + it) * MD_STEP;
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int r = 0; r < 4; ++r)
              if (t0 + 16 * h + 4 * g + r >= CL_SKV) st[t][h][r] = CL_NEG_BIG;      // weight exp2(-huge) = 0
      }
      float mx[2], alpha[2] = {1.0f, 1.0f};
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        const float lo = fmaxf(fmaxf(st[t][0][0], st[t][0][1]), fmaxf(st[t][0][2], st[t][0][3]));
        const float hi = fmaxf(fmaxf(st[t][1][0], st[t][1][1]), fmaxf(st[t][1][2], st[t][1][3]));
        mx[t] = fmaxf(lo, hi) * CL_SCALE_LOG2E;
      }
      if (it == 0 || __builtin_amdgcn_ballot_w64(mx[0] > m_run[0] + MD_RESCALE_STEP || mx[1] > m_run[1] + MD_RESCALE_STEP)) {
        // cold after the first step: each head's largest score of this step over all four lane groups
#pragma unroll
        for (int t = 0; t < 2; ++t) {
          float v = mx[t];
          v = fmaxf(v, lane_xor(v, lane, 16));
          v = fmaxf(v, lane_xor(v, lane, 32));
          if (it == 0) {
            m_run[t] = v;                           // nothing accumulated yet: the step's own maximum
          } else if (v > m_run[t] + MD_RESCALE_STEP) {
            alpha[t] = fast_exp2(m_run[t] - v);
            m_run[t] = v;
            l_acc[t] *= alpha[t];
          }
        }
      }
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        elem8 pf;
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
          for (int r = 0; r < 4; ++r)
            pf[4 * h + r] = to_elem(fast_exp2(__builtin_fmaf(st[t][h][r], CL_SCALE_LOG2E, -m_run[t])));
        md_weights[it & 1][set][t][lane] = as_u32x4(pf);
        md_alpha[it & 1][set][t][lane] = alpha[t];
        l_acc[t] = mfma16(ones, pf, l_acc[t]);      // row sums of exactly the rounded weights
      }
    }
    if (g == 0) {
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        md_final[set][t][0][c] = m_run[t];
        md_final[set][t][1][c] = l_acc[t][0];
      }
    }
    md_barrier();                                   // (m, l) are there for the value waves
    return;
  }

  // ============================================================================= value wave
  // loads of step index s (relative to the split), clamped onto the split's last step so that the
  // load counter holds the same number of steps at every wait
  u32 lat_off, pe_off;
  {
    const int r = 8 * loader + (lane >> 3);
    const int chunk = (lane & 7) ^ md_swz(r);
    lat_off = (u32)((r * CL_CKV + 8 * chunk) * 2);
    pe_off = (u32)((r * CL_KPE + 8 * chunk) * 2);
  }
  auto issue = [&](int s) __attribute__((always_inline)) {
#ifdef CL_DBG_NODMA
    return;
#endif
    int rel = s < n_own - 1 ? s : n_own - 1;
    rel = rel > 0 ? rel : 0;
    const int t0 = (step_begin + rel) * MD_STEP;
    md_issue_from<0>(lat_off, pe_off, kv + (i64)t0 * CL_CKV, kpe + (i64)t0 * CL_KPE, t0,
                     tiles_byte + (unsigned)((s % MD_STAGES) * MD_TILE * 2), loader);
  };
  f32x4 acc[2][MD_FBW];                             // acc[t][fb][r] = O[head 16 t + c][16 (FBW fhalf + fb) + 4 g + r]
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int fb = 0; fb < MD_FBW; ++fb) acc[t][fb] = (f32x4){0.f, 0.f, 0.f, 0.f};
  const int vtok = 4 * g + (c >> 2);
  const int v_lo = fhalf * (MD_FBW / 4) * MD_PANEL + vtok * 64 + (((((c & 3) >> 1)) ^ md_swz(vtok)) << 3) + 4 * (c & 1);

  if (n_own > 0) {
    issue(0);
    issue(1);
  }
  for (int it = 0; it <= n_own; ++it) {
    // image `it` must have landed before the barrier lets the score waves read it: at most the
    // loads of image it + 1 may be outstanding (none are issued for an empty split)
    if (n_own > 0) __builtin_amdgcn_s_waitcnt(0x0F70 | (MD_UNITS_PER & 15) | ((MD_UNITS_PER >> 4) << 14));
    md_barrier();
    if (it < n_own) issue(it + 2);                  // into the slot image it - 2 has left
    if (it == 0) continue;
    const elem_t* tile = md_tiles + ((it - 1) % MD_STAGES) * MD_TILE;
#ifdef CL_DBG_NOV
    continue;
#endif
    elem8 pf[2];
    float alpha[2];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      pf[t] = as_elem8(md_weights[(it - 1) & 1][set][t][lane]);
      alpha[t] = md_alpha[(it - 1) & 1][set][t][lane];
    }
    if (__builtin_amdgcn_ballot_w64(alpha[0] != 1.0f || alpha[1] != 1.0f)) {
      // cold: the score wave raised a reference point at this step
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int fb = 0; fb < MD_FBW; ++fb) acc[t][fb] *= alpha[t];
    }
    // out^T block fb: rows = features 16 fb + (0..15), slots = tokens 4 g + (0..3), 16 + 4 g + (0..3)
#pragma unroll
    for (int fb = 0; fb < MD_FBW; ++fb) {
      const elem_t* p = tile + (fb >> 2) * MD_PANEL + (v_lo ^ (((2 * fb) & 7) << 3));
      const md_s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((md_lds_s16x4*)(p));
      const md_s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((md_lds_s16x4*)(p + 16 * 64));
      const elem8 a = __builtin_bit_cast(elem8, (md_s16x8)__builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
#pragma unroll
      for (int t = 0; t < 2; ++t) acc[t][fb] = mfma16(a, pf[t], acc[t][fb]);
    }
    __builtin_amdgcn_sched_group_barrier(0x100, CL_LDS_AHEAD, 0);
#pragma unroll
    for (int n = 0; n < MD_FBW - CL_LDS_AHEAD / 2; ++n) {
      __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
    }
    __builtin_amdgcn_sched_group_barrier(0x008, CL_LDS_AHEAD, 0);
  }
  __builtin_amdgcn_s_waitcnt(0x0F70);               // no load may still be on its way into LDS when the workgroup ends
  md_barrier();                                     // the score waves have left (m, l)

  // ---- this wave writes its half of the features of its head set --------------------------------
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    const float m = md_final[set][t][0][c], l = md_final[set][t][1][c];
    const i64 orow = row0 + 16 * t + c;
    const int f0 = 16 * MD_FBW * fhalf + 4 * g;
#if CL_SPLITS > 1 && !CL_PO_ELEM
    const i64 prow = (i64)split * CL_TOTAL_ROWS + orow;
#pragma unroll
    for (int fb = 0; fb < MD_FBW; ++fb) *reinterpret_cast<f32x4*>(CL_ARG_PO + prow * CL_CKV + f0 + 16 * fb) = acc[t][fb];
    if (g == 0 && fhalf == 0) {
      CL_ARG_PM[prow] = m;
      CL_ARG_PL[prow] = l;
    }
#else
    const float inv = 1.0f / fmaxf(l, 1.0e-30f);
#if CL_SPLITS > 1
    const i64 prow = (i64)split * CL_TOTAL_ROWS + orow;
    elem_t* dst_row = CL_ARG_PO + prow * CL_CKV;
    if (g == 0 && fhalf == 0) {
      CL_ARG_PM[prow] = l > 0.f ? m + fast_log2(l) : CL_NEG_BIG;
      CL_ARG_PL[prow] = l > 0.f ? 1.0f : 0.f;
    }
#else
    elem_t* dst_row = CL_ARG_OUT + orow * CL_CKV;
#if CL_EMIT_LSE
    if (g == 0 && fhalf == 0) CL_ARG_LSE[orow] = l > 0.f ? m + fast_log2(l) : CL_NEG_INF;
#endif
#endif
#pragma unroll
    for (int fb = 0; fb < MD_FBW; ++fb) {
      elem4 y;
#pragma unroll
      for (int r = 0; r < 4; ++r) y[r] = to_elem(acc[t][fb][r] * inv);
      *reinterpret_cast<elem4*>(dst_row + f0 + 16 * fb) = y;
    }
#endif
  }
}
#endif  // CL_EMIT_PARTIAL
