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
// have.  Two kinds of wave do, eight waves for 64 heads:
//
//   score wave (s, h) (4)       keeps the Q fragments of heads 32 s .. 32 s + 31 and makes their
//                               scores against tokens 16 h .. 16 h + 15 of every step; every key
//                               fragment it reads feeds two matrix ops (its two head tiles).  It
//                               turns them into weights against reference points of its own (one
//                               per head) and leaves the weights (its half of the value product's
//                               B operand, 8 bytes per lane and head tile) and the reference
//                               points it used in LDS;
//   value wave (s, f) (4)       keeps the accumulators of the same 32 heads for half of the
//                               latent features (2 x 16 x 16 x 16 values), the weight sums and the
//                               reference points the accumulators stand against; every value
//                               fragment it reads feeds two matrix ops.  It picks the weights of
//                               step t - 1 up and adds their value product.  The value waves also
//                               issue every tile load and write the result.
//
// Per step and 64 heads that is 72 + 72 KB out of LDS for 280 matrix ops.  Every SIMD holds one
// score wave and one value wave (wave w runs on SIMD w % 4): 70 matrix ops per SIMD and step, and
// what a score wave does outside the matrix unit -- wait for its first key fragments after the
// barrier, then maxima, exponentials and the hand-over, a third of its step -- runs under the
// value wave's matrix ops (measured: 0.90 us per step against 1.0 with the score waves paired on
// two SIMDs and the value waves on the other two).  The loop is skewed by one step, one barrier
// per step: in iteration t the score waves read image t and the value waves image t - 1, the
// loads of images t + 1 and t + 2 are in flight (four images).  A value wave reads the operands
// of its first feature blocks of image t at the end of iteration t, across the barrier, and asks
// for the panels of image t + 2 between its matrix ops.
//
// Ends of the kernel.  The 64 heads' Q rows reach the score waves through LDS (whole 1 KiB runs
// into the LDS of the two images loaded last; read straight from global memory a fragment is
// sixteen 64-byte pieces per instruction and both token halves would fetch the same rows: 3 us
// more before the first step at 16 x 128 heads), and the value waves' results leave as 16-byte
// pieces after a row swap between lane groups (as the 8-byte pieces the accumulators hold they
// took 2 us longer).
//
// Softmax reference points without a handshake.  A score wave raises a head's reference point
// only when a score of its own tokens passes it by 2^8, so its weights never exceed 2^8; with
// each step's weights it publishes the points it used, and one step later adopts the other token
// half's points where those are higher (a maximum, nothing to rescale: score waves keep no
// sums).  The value waves compare the two published points of a step with the point their
// accumulators stand against: equal on ordinary steps; otherwise (cold) they take the highest
// of the three, scale accumulators and sums by 2^(old - new) and the weights of a token half
// that used a lower point by 2^(its - new), rounded to 16 bits again (the sums are taken over the
// weights as used).
//
//   CL_HEADS (multiple of 64)  CL_CKV (multiple of 128)  CL_KPE (multiple of 64)  CL_SKV  CL_BATCH
//   CL_SPLITS  CL_SCALE_LOG2E  CL_PO_ELEM (must be 1: split partials normalised, in the element type)

#if CL_SPLITS > 1 && !CL_PO_ELEM
#error "the score-wave / value-wave kernel writes its split partials in the element type"
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
#define MD_THREADS 512
#define MD_HEADS_PER_BLOCK 64
#define MD_HEAD_GROUPS (CL_HEADS / MD_HEADS_PER_BLOCK)
#define MD_UNITS_PER MD_PANELS                  // 1 KiB loads per value wave and step: its 8-token group of every panel
#define MD_RESCALE_STEP 8.0f
#define MD_QCHUNKS (MD_D / 8)                    // 16-byte chunks of one head's Q row (latent + rope)
#define MD_REF_FLOOR (-1.0e20f)                   // lowest reference point: a token half with every token masked stands here
#ifndef CL_LDS_AHEAD
#define CL_LDS_AHEAD 8
#endif
#ifndef CL_S_AHEAD
#define CL_S_AHEAD CL_LDS_AHEAD                 // key fragments a score wave asks for ahead of its matrix ops
#endif
#ifndef CL_S_PANELS
#define CL_S_PANELS 0                           // panels of every image (from the third on) the score waves ask for
#endif
#define MD_V_UNITS (MD_PANELS - CL_S_PANELS)    // loads per value wave and step once the score waves share them
static_assert(CL_S_PANELS >= 0 && CL_S_PANELS < MD_PANELS, "the value waves keep at least one panel");
static_assert(CL_CKV % 128 == 0 && CL_KPE % 64 == 0, "whole 64-feature panels, the latent ones halved between two value waves");
static_assert(CL_HEADS % MD_HEADS_PER_BLOCK == 0, "64 heads per workgroup");
static_assert(CL_SCALE_LOG2E > 0.f, "the largest raw score must be the largest scaled one");
static_assert(MD_UNITS_PER < 32, "load counter range");
static_assert(MD_FBW % 2 == 0, "a value wave's feature blocks leave in pairs");
constexpr bool MD_RAGGED = CL_SKV % MD_STEP != 0;

__shared__ __attribute__((aligned(1024))) elem_t md_tiles[MD_STAGES * MD_TILE];
// [step parity][head set][head tile][token half][lane]: the lane's four weights of each token half.  A
// score wave writes 8 bytes per lane side by side (lanes 16 bytes apart, the two halves interleaved,
// put lanes l and l + 16 into the same banks); a value wave reads its lane's two halves as two
// 8-byte pieces.
__shared__ __attribute__((aligned(16))) u32x2 md_weights[2][2][2][2][64];
// [step parity][head set][head tile][head][token half]: the reference point those weights stand against
__shared__ __attribute__((aligned(8))) float md_ref[2][2][2][16][2];

typedef short md_s16x4 __attribute__((ext_vector_type(4)));
typedef short md_s16x8 __attribute__((ext_vector_type(8)));
typedef __attribute__((address_space(3))) md_s16x4 md_lds_s16x4;

CL_DEVICE int md_swz(int token) { return token & 6; }

// rows (16 lanes) 1 and 3 of `a` trade places with rows 0 and 2 of `b`
CL_DEVICE void md_swap_rows16(unsigned& a, unsigned& b) {
  asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 0" : "+v"(a), "+v"(b));
}

// x with bits 0 and 3 trading places
CL_DEVICE int md_trade03(int x) { return (x & ~9) | ((x & 1) << 3) | ((x >> 3) & 1); }
static_assert(MD_QCHUNKS % 16 == 8, "the Q rows in LDS: a row's parity moves it by eight 16-byte bank groups");

// 16 bytes per lane, global -> LDS; not counted by the compiler, the issuing wave waits itself
template <int OFF>
CL_DEVICE void md_dma16(const void* gptr, unsigned lds_byte) {
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off offset:%2"
               :: "v"(gptr), "s"(__builtin_amdgcn_readfirstlane(lds_byte)), "n"(OFF) : "memory", "m0");
}

// the same between the matrix ops of a loop body: without the compiler-level memory barrier (the
// slot written is one no wave reads before the next workgroup barrier), so LDS reads may still be
// scheduled across it
CL_DEVICE void md_dma16_loose(const void* gptr, unsigned lds_byte) {
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
               :: "v"(gptr), "s"(__builtin_amdgcn_readfirstlane(lds_byte)) : "m0");
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

// value wave `lw`: its load of panel `p` of one step (p constant after unrolling)
CL_DEVICE void md_issue_panel(int p, u32 lat_off, u32 pe_off, const elem_t* lat_rows, const elem_t* pe_rows, int t0,
                              unsigned stage_byte, int lw) {
  const unsigned lds_byte = stage_byte + (unsigned)(p * MD_PANEL * 2 + lw * 1024);
  const bool lat = p < MD_LAT_PANELS;
  const int col = 64 * (lat ? p : p - MD_LAT_PANELS);
  if (MD_RAGGED) {
    const int lane = threadIdx.x & 63;
    const int r = 8 * lw + (lane >> 3);
    int t = t0 + r;
    t = t < CL_SKV - 1 ? t : CL_SKV - 1;
    const int chunk = (lane & 7) ^ md_swz(r);
    md_dma16_loose(lat ? lat_rows + (i64)(t - t0) * CL_CKV + col + 8 * chunk : pe_rows + (i64)(t - t0) * CL_KPE + col + 8 * chunk,
                   lds_byte);
  } else {
    md_dma16_loose(lat ? reinterpret_cast<const char*>(lat_rows + col) + lat_off
                       : reinterpret_cast<const char*>(pe_rows + col) + pe_off, lds_byte);
  }
}
#if CL_EMIT_PARTIAL
extern "C" __global__ void __launch_bounds__(MD_THREADS)
CL_PARTIAL_NAME(CL_PARTIAL_PARAMS) {
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int c = lane & 15, g = lane >> 4;
  // waves 0..3: score waves, waves 4..7: value waves; of both, wave w has head set w % 2 and
  // token half (score) or feature half (value) (w / 2) % 2.  Wave w runs on SIMD w % 4: one score
  // wave and one value wave on every SIMD.
  const bool scores = wave < 4;
  const int set = wave & 1;
  const int fhalf = (wave >> 1) & 1;                      // score waves: the token half
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

  // The Q rows of the 64 heads go through LDS: every wave asks for its share as whole 1 KiB runs
  // (64 consecutive 16-byte slots each), into the two images' worth of LDS the loop fills last;
  // row n / MD_QCHUNKS holds the head whose number is the row's with bits 0 and 3 traded, and slot
  // n % MD_QCHUNKS of it the 16-byte chunk whose low three bits are the slot's XOR head % 8.  A
  // fragment read has the sixteen heads of a tile side by side: the XOR spreads heads that differ
  // in their low three bits over eight 16-byte bank groups, and since a row is an odd multiple of
  // eight such groups long, the row's parity -- bit 3 of the head -- picks the other eight for
  // heads c and c + 8 (with rows in head order they met in the same banks).  Read straight from
  // global memory, a fragment is sixteen 64-byte pieces per instruction, and both token halves
  // would fetch the same rows.
  if (n_own > 0) {
    const i64 wg_row0 = (i64)b * CL_HEADS + hg_block * MD_HEADS_PER_BLOCK;
    for (int k = wave; k < MD_QCHUNKS; k += MD_THREADS / 64) {       // 64 heads x MD_QCHUNKS slots = MD_QCHUNKS runs
      const int n = 64 * k + lane;
      const int row = n / MD_QCHUNKS, pos = n % MD_QCHUNKS;
      const int h = md_trade03(row);
      const int q = (pos & ~7) | ((pos ^ h) & 7);
      const elem_t* src = q < CL_CKV / 8 ? CL_ARG_Q + (wg_row0 + h) * CL_CKV + 8 * q
                                         : CL_ARG_QPE + (wg_row0 + h) * CL_KPE + 8 * (q - CL_CKV / 8);
      md_dma16<0>(src, tiles_byte + (unsigned)(2 * MD_TILE * 2 + 1024 * k));
    }
  }
  // this wave's piece of every panel it loads: token rows 8 loader + lane / 8, the chunk that belongs in slot lane % 8
  u32 lat_off, pe_off;
  {
    const int r = 8 * loader + (lane >> 3);
    const int chunk = (lane & 7) ^ md_swz(r);
    lat_off = (u32)((r * CL_CKV + 8 * chunk) * 2);
    pe_off = (u32)((r * CL_KPE + 8 * chunk) * 2);
  }
  if (scores) {
    // =========================================================================== score wave
    // Q fragments (B operand): lane (c, g) holds q[head 16 t + c][32 j + 8 g .. + 8] for head tile t
    elem8 qf[2][MD_KJ];
    if (n_own > 0) {
      __builtin_amdgcn_s_waitcnt(0x0F70);             // this wave's runs have landed
      md_barrier();                                   // and everybody else's
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int j = 0; j < MD_KJ; ++j) {
          const int row = 32 * set + 16 * t + md_trade03(c), q = 4 * j + g;
          qf[t][j] = *reinterpret_cast<const elem8*>(md_tiles + 2 * MD_TILE + (row * MD_QCHUNKS + ((q & ~7) | ((q ^ c) & 7))) * 8);
        }
    } else {
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int j = 0; j < MD_KJ; ++j) qf[t][j] = (elem8){};
    }
    float m_run[2] = {CL_NEG_BIG, CL_NEG_BIG};      // reference point of head c of each tile (log2 domain), uniform over g
    const int half = fhalf;
    const int a_lo = (16 * half + c) * 64 + ((g ^ md_swz(c)) << 3);

    for (int it = 0; it <= n_own; ++it) {
#if CL_S_PANELS
      // this wave's panels of image `it` have landed: at most those of image it + 1 are on their way
      __builtin_amdgcn_s_waitcnt(0x0F70 | (CL_S_PANELS & 15));
#endif
      md_barrier();                                 // image `it` has landed (the value waves waited for it)
      if (it == n_own) break;
      const elem_t* tile = md_tiles + (it % MD_STAGES) * MD_TILE;
      // the points the other token half used one step ago: asked for first, so that the answer is
      // there when the matrix ops are done
      float other[2] = {CL_NEG_BIG, CL_NEG_BIG};
      if (it > 0) {
#pragma unroll
        for (int t = 0; t < 2; ++t) other[t] = md_ref[(it - 1) & 1][set][t][c][half ^ 1];
      }
      __builtin_amdgcn_sched_barrier(0);
      // scores^T: rows = tokens 16 half + (0..15), columns = heads of tile t; even and odd
      // 32-feature slices in accumulators of their own
      f32x4 sp[2][2];
#pragma unroll
      for (int t = 0; t < 2; ++t) sp[t][0] = sp[t][1] = (f32x4){0.f, 0.f, 0.f, 0.f};
#if CL_S_PANELS
      // this wave's share of the loads of image it + 2, from the second iteration on (the value
      // waves ask for images 0 to 2 whole); past the split's end as in the value waves
      const int ahead = it + 2 < n_own + 1 ? it + 2 : n_own + 1;
      const int rel = ahead < n_own - 1 ? ahead : n_own - 1;
      const int t0_ahead = (step_begin + rel) * MD_STEP;
      const elem_t* lat_rows = kv + (i64)t0_ahead * CL_CKV;
      const elem_t* pe_rows = kpe + (i64)t0_ahead * CL_KPE;
      const unsigned stage_byte = tiles_byte + (unsigned)((ahead % MD_STAGES) * MD_TILE * 2);
#endif
#pragma unroll
      for (int j = 0; j < MD_KJ; ++j) {
        const elem8 a = *reinterpret_cast<const elem8*>(tile + (j >> 1) * MD_PANEL + (a_lo ^ ((4 * (j & 1)) << 3)));
#pragma unroll
        for (int t = 0; t < 2; ++t) sp[t][j & 1] = mfma16(a, qf[t][j], sp[t][j & 1]);
#if CL_S_PANELS
        if (it > 0) {
#pragma unroll
          for (int pn = 0; pn < CL_S_PANELS; ++pn)
            if ((pn * MD_KJ) / CL_S_PANELS == j) md_issue_panel(pn, lat_off, pe_off, lat_rows, pe_rows, t0_ahead, stage_byte, loader);
        }
#endif
      }
      __builtin_amdgcn_sched_group_barrier(0x100, CL_S_AHEAD, 0);
#pragma unroll
      for (int n = 0; n < MD_KJ - CL_S_AHEAD; ++n) {
        __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      }
      __builtin_amdgcn_sched_group_barrier(0x008, 2 * CL_S_AHEAD, 0);
      f32x4 st[2];
#pragma unroll
      for (int t = 0; t < 2; ++t) st[t] = sp[t][0] + sp[t][1];

      if (MD_RAGGED) {
        const int t0 = (step_begin + it) * MD_STEP + 16 * half + 4 * g;
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int r = 0; r < 4; ++r)
            if (t0 + r >= CL_SKV) st[t][r] = CL_NEG_BIG;      // weight exp2(-huge) = 0
      }
      float mx[2];
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        mx[t] = fmaxf(fmaxf(st[t][0], st[t][1]), fmaxf(st[t][2], st[t][3])) * CL_SCALE_LOG2E;
        m_run[t] = fmaxf(m_run[t], other[t]);         // adopted where higher
      }
      if (it == 0 || __builtin_amdgcn_ballot_w64(mx[0] > m_run[0] + MD_RESCALE_STEP || mx[1] > m_run[1] + MD_RESCALE_STEP)) {
        // cold after the first step: each head's largest score of this step over all four lane groups
#pragma unroll
        for (int t = 0; t < 2; ++t) {
          float v = mx[t];
          v = fmaxf(v, lane_xor(v, lane, 16));
          v = fmaxf(v, lane_xor(v, lane, 32));
          if (it == 0)
            m_run[t] = fmaxf(v, MD_REF_FLOOR);      // nothing behind it yet: the step's own maximum
          else if (v > m_run[t] + MD_RESCALE_STEP)
            m_run[t] = v;
        }
      }
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        elem4 pf;
#pragma unroll
        for (int r = 0; r < 4; ++r) pf[r] = to_elem(fast_exp2(__builtin_fmaf(st[t][r], CL_SCALE_LOG2E, -m_run[t])));
        md_weights[it & 1][set][t][half][lane] = __builtin_bit_cast(u32x2, pf);
        if (g == 0) md_ref[it & 1][set][t][c][half] = m_run[t];
      }
    }
#if CL_S_PANELS
    __builtin_amdgcn_s_waitcnt(0x0F70);             // no load may still be on its way into LDS when the workgroup ends
#endif
    return;
  }

  // ============================================================================= value wave
  // loads of step index s (relative to the split), clamped onto the split's last step so that the
  // load counter holds the same number of steps at every wait
  auto issue = [&](int s) __attribute__((always_inline)) {
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
  elem8 ones;
#pragma unroll
  for (int i = 0; i < 8; ++i) ones[i] = to_elem(1.0f);
  f32x4 l_acc[2];                                   // every component: sum of the weights of head c (both feature halves keep it)
  l_acc[0] = l_acc[1] = (f32x4){0.f, 0.f, 0.f, 0.f};
  float m_acc[2] = {CL_NEG_BIG, CL_NEG_BIG};        // the reference point accumulators and sums stand against
  const int vtok = 4 * g + (c >> 2);
  const int v_lo = fhalf * (MD_FBW / 4) * MD_PANEL + vtok * 64 + (((((c & 3) >> 1)) ^ md_swz(vtok)) << 3) + 4 * (c & 1);

  if (n_own > 0) {
    issue(0);
    issue(1);
    // this wave's Q runs (asked for before the two images) have landed, then everybody else's
    __builtin_amdgcn_s_waitcnt(0x0F70 | ((2 * MD_UNITS_PER) & 15) | (((2 * MD_UNITS_PER) >> 4) << 14));
    md_barrier();
  }
  // the value operands of the first MD_PRE feature blocks of the next image: read at the end of an
  // iteration, they are on their way while the waves meet at the barrier
  constexpr int MD_PRE = CL_LDS_AHEAD / 2;
  static_assert(MD_PRE >= 1 && MD_FBW % MD_PRE == 0, "the read-ahead operands are a ring the feature blocks walk whole turns of");
  md_s16x4 pre_lo[MD_PRE], pre_hi[MD_PRE];
#pragma unroll
  for (int fb = 0; fb < MD_PRE; ++fb) pre_lo[fb] = pre_hi[fb] = (md_s16x4){0, 0, 0, 0};
  auto operand = [&](const elem_t* tile, int fb, md_s16x4& lo, md_s16x4& hi) __attribute__((always_inline)) {
    const elem_t* p = tile + (fb >> 2) * MD_PANEL + (v_lo ^ (((2 * fb) & 7) << 3));
    lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((md_lds_s16x4*)(p));
    hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((md_lds_s16x4*)(p + 16 * 64));
  };
  for (int it = 0; it <= n_own; ++it) {
    // image `it` must have landed before the barrier lets the score waves read it: at most the
    // loads of image it + 1 may be outstanding (none are issued for an empty split)
    // (with the score waves sharing the loads the later images are MD_V_UNITS loads each: waiting
    // down to that count is the right wait for them and a longer one for the first three)
    if (n_own > 0) __builtin_amdgcn_s_waitcnt(0x0F70 | (MD_V_UNITS & 15) | ((MD_V_UNITS >> 4) << 14));
    md_barrier();
    const elem_t* next_tile = md_tiles + (it % MD_STAGES) * MD_TILE;           // image `it`: there from here on
    if (it == 0) {
      if (it < n_own) issue(it + 2);
#pragma unroll
      for (int fb = 0; fb < MD_PRE; ++fb) operand(next_tile, fb, pre_lo[fb], pre_hi[fb]);
      continue;
    }
    const elem_t* tile = md_tiles + ((it - 1) % MD_STAGES) * MD_TILE;
    elem8 pf[2];
    f32x2 ref[2];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      {
        const u32x2 lo2 = md_weights[(it - 1) & 1][set][t][0][lane], hi2 = md_weights[(it - 1) & 1][set][t][1][lane];
        pf[t] = as_elem8((u32x4){lo2[0], lo2[1], hi2[0], hi2[1]});
      }
      ref[t] = *reinterpret_cast<const f32x2*>(&md_ref[(it - 1) & 1][set][t][c][0]);
    }
    if (__builtin_amdgcn_ballot_w64(ref[0][0] != m_acc[0] || ref[0][1] != m_acc[0] || ref[1][0] != m_acc[1] ||
                                    ref[1][1] != m_acc[1])) {
      // cold: a score wave raised a reference point at this step (or this is the first step)
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        const float m_new = fmaxf(ref[t][0], ref[t][1]);          // never below m_acc
        const float alpha = fast_exp2(m_acc[t] - m_new);
        const float f_lo = fast_exp2(ref[t][0] - m_new), f_hi = fast_exp2(ref[t][1] - m_new);
        m_acc[t] = m_new;
#pragma unroll
        for (int fb = 0; fb < MD_FBW; ++fb) acc[t][fb] *= alpha;
        l_acc[t] *= alpha;
#pragma unroll
        for (int i = 0; i < 8; ++i) pf[t][i] = to_elem(to_f32(pf[t][i]) * (i < 4 ? f_lo : f_hi));
      }
    }
    // The loads of image it + 2 (into the slot image it - 2 has left) are asked for between the
    // matrix ops, panel p after feature block p * MD_FBW / MD_PANELS.  Past the split's end the
    // last image is asked for again, into the slot of image n_own + 1 (which holds or awaits the
    // same rows): the load counter then holds the same number of loads at every wait.
    const int ahead = it + 2 < n_own + 1 ? it + 2 : n_own + 1;
    const int rel = ahead < n_own - 1 ? ahead : n_own - 1;
    const int t0 = (step_begin + rel) * MD_STEP;
    const elem_t* lat_rows = kv + (i64)t0 * CL_CKV;
    const elem_t* pe_rows = kpe + (i64)t0 * CL_KPE;
    const unsigned stage_byte = tiles_byte + (unsigned)((ahead % MD_STAGES) * MD_TILE * 2);
    // out^T block fb: rows = features 16 fb + (0..15), slots = tokens 4 g + (0..3), 16 + 4 g + (0..3)
#pragma unroll
    for (int fb = 0; fb < MD_FBW; ++fb) {
      md_s16x4 lo = pre_lo[fb % MD_PRE], hi = pre_hi[fb % MD_PRE];
      const elem8 a = __builtin_bit_cast(elem8, (md_s16x8)__builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
#pragma unroll
      for (int t = 0; t < 2; ++t) acc[t][fb] = mfma16(a, pf[t], acc[t][fb]);
      // the operand MD_PRE blocks on: of this image, or (the last MD_PRE) of the next one
      if (fb + MD_PRE < MD_FBW)
        operand(tile, fb + MD_PRE, pre_lo[fb % MD_PRE], pre_hi[fb % MD_PRE]);
      else
        operand(next_tile, fb + MD_PRE - MD_FBW, pre_lo[fb % MD_PRE], pre_hi[fb % MD_PRE]);
#pragma unroll
      for (int pn = CL_S_PANELS; pn < MD_PANELS; ++pn)
        if (((pn - CL_S_PANELS) * MD_FBW) / MD_V_UNITS == fb) md_issue_panel(pn, lat_off, pe_off, lat_rows, pe_rows, t0, stage_byte, loader);
    }
#pragma unroll
    for (int n = 0; n < MD_FBW; ++n) {
      __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
    }
#pragma unroll
    for (int t = 0; t < 2; ++t) l_acc[t] = mfma16(ones, pf[t], l_acc[t]);      // row sums of exactly the weights used
  }
  __builtin_amdgcn_s_waitcnt(0x0F70);               // no load may still be on its way into LDS when the workgroup ends

  // ---- this wave writes its half of the features of its head set --------------------------------
  // A lane holds features 16 fb + 4 g .. + 3 of its head for every block fb of the wave's half.
  // Lanes g and g ^ 1 trade halves of a pair of blocks (one row swap per register), so that each
  // stores 16 contiguous bytes and a store instruction covers 64 contiguous bytes of sixteen rows:
  // even g the 8 features from 4 g of the even block, odd g those from 4 (g - 1) of the odd one.
  // (Before: the rows went through LDS so that a store covered whole half rows; the paired 8-byte
  // LDS writes of that staging were the kernel's remaining bank conflicts.)
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    const float m = m_acc[t], l = l_acc[t][0];
    const i64 orow = row0 + 16 * t;                                // first head row of this tile
    const float inv = 1.0f / fmaxf(l, 1.0e-30f);
#if CL_SPLITS > 1
    const i64 prow = (i64)split * CL_TOTAL_ROWS + orow;
    elem_t* dst = CL_ARG_PO + (prow + c) * CL_CKV + 16 * MD_FBW * fhalf + 16 * (g & 1) + 4 * (g & 2);
    if (g == 0 && fhalf == 0) {
      CL_ARG_PM[prow + c] = l > 0.f ? m + fast_log2(l) : CL_NEG_BIG;
      CL_ARG_PL[prow + c] = l > 0.f ? 1.0f : 0.f;
    }
#else
    elem_t* dst = CL_ARG_OUT + (orow + c) * CL_CKV + 16 * MD_FBW * fhalf + 16 * (g & 1) + 4 * (g & 2);
#if CL_EMIT_LSE
    if (g == 0 && fhalf == 0) CL_ARG_LSE[orow + c] = l > 0.f ? m + fast_log2(l) : CL_NEG_INF;
#endif
#endif
#pragma unroll
    for (int fp = 0; fp < MD_FBW / 2; ++fp) {
      elem4 y0, y1;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        y0[r] = to_elem(acc[t][2 * fp][r] * inv);
        y1[r] = to_elem(acc[t][2 * fp + 1][r] * inv);
      }
      const u32x2 a = __builtin_bit_cast(u32x2, y0), b = __builtin_bit_cast(u32x2, y1);
      unsigned a0 = a[0], a1 = a[1], b0 = b[0], b1 = b[1];
      md_swap_rows16(a0, b0);
      md_swap_rows16(a1, b1);
      *reinterpret_cast<u32x4*>(dst + 32 * fp) = (u32x4){a0, a1, b0, b1};
    }
  }
}
#endif  // CL_EMIT_PARTIAL
