// ---- shared device helpers (gfx950: wave64, MFMA 16x16x32 f16/bf16) ------------------------
// Element type is chosen by the emitter: CL_BF16 == 1 selects bfloat16, else half.
#if CL_BF16
typedef __bf16 elem_t;
#else
typedef _Float16 elem_t;
#endif
typedef elem_t elem8 __attribute__((ext_vector_type(8)));
typedef elem_t elem4 __attribute__((ext_vector_type(4)));
typedef elem_t elem2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef unsigned int u32;
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
typedef long long i64;

#define CL_DEVICE static __device__ __forceinline__
#define CL_METHOD __device__ __forceinline__
#define CL_NEG_BIG (-1.0e30f)
#define CL_NEG_INF (__builtin_bit_cast(float, 0xff800000u))

// D(16x16 f32) += A(16x32) * B(32x16).  Lane l supplies A[row l%16][k-slots of group l/16] and
// B[k-slots of group l/16][col l%16]; it receives D[rows 4*(l/16)+0..3][col l%16].  A and B are
// paired slot by slot, so any consistent assignment of the contraction index to slots works.
CL_DEVICE f32x4 mfma16(elem8 a, elem8 b, f32x4 c) {
#if CL_BF16
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
#else
  return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
#endif
}

CL_DEVICE float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
CL_DEVICE float fast_log2(float x) { return __builtin_amdgcn_logf(x); }
CL_DEVICE float fast_rsqrt(float x) { return __builtin_amdgcn_rsqf(x); }
CL_DEVICE float fast_rcp(float x) { return __builtin_amdgcn_rcpf(x); }

// Value of `v` held by lane (lane ^ mask); mask is a compile-time constant < 64.
CL_DEVICE float lane_xor(float v, int lane, int mask) {
  return __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute((lane ^ mask) << 2, __builtin_bit_cast(int, v)));
}
CL_DEVICE float lane_read(float v, int src_lane) {
  return __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(src_lane << 2, __builtin_bit_cast(int, v)));
}

// Search of a row-pointer array (batch + 1 non-decreasing entries, clamped into [0, limit]) by
// all lanes of a wave at once: the last request b of [0, batch) with
//   with_b * b + ptr[b] / div <= item
// (true for every request up to that one, so the lanes test 64 requests at a time and count:
// one round trip to memory per 256 requests where a bisection makes one per halving), and the
// clamped ptr[b], ptr[b + 1] -- out of the lanes when there are fewer than 64 requests.
struct ClRequest { int req, p0, p1, s0, s1; };   // s0, s1: the same two entries of a second pointer array
CL_DEVICE int cl_clamp_ptr(int p, int limit) { return p < 0 ? 0 : (p > limit ? limit : p); }
// `second` (may be null): another row-pointer array of the same requests, clamped into [0, limit2];
// its entries for the request found come back as s0, s1 -- read in the same round trip as the
// searched array when there are fewer than 64 requests.
CL_DEVICE ClRequest cl_find_request(const int* __restrict__ ptr, int batch, int limit, int div, int with_b,
                                    int item, int lane, const int* __restrict__ second = nullptr, int limit2 = 0) {
  const int v0 = cl_clamp_ptr(ptr[lane < batch ? lane : batch], limit);
  const int w0 = second ? cl_clamp_ptr(second[lane < batch ? lane : batch], limit2) : 0;
  int count = __builtin_popcountll(__builtin_amdgcn_ballot_w64(lane < batch && with_b * lane + v0 / div <= item));
  for (int base = 64; base < batch; base += 256) {
    int v[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int b = base + 64 * k + lane;
      v[k] = cl_clamp_ptr(ptr[b < batch ? b : batch], limit);
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int b = base + 64 * k + lane;
      count += __builtin_popcountll(__builtin_amdgcn_ballot_w64(b < batch && with_b * b + v[k] / div <= item));
    }
  }
  ClRequest r;
  r.req = count > 0 ? count - 1 : 0;
  r.s0 = r.s1 = 0;
  if (batch < 64) {
    r.p0 = __builtin_amdgcn_readlane(v0, r.req);
    r.p1 = __builtin_amdgcn_readlane(v0, r.req + 1);
    r.s0 = __builtin_amdgcn_readlane(w0, r.req);
    r.s1 = __builtin_amdgcn_readlane(w0, r.req + 1);
  } else {
    r.p0 = cl_clamp_ptr(ptr[r.req], limit);
    r.p1 = cl_clamp_ptr(ptr[r.req + 1], limit);
    if (second) {
      r.s0 = cl_clamp_ptr(second[r.req], limit2);
      r.s1 = cl_clamp_ptr(second[r.req + 1], limit2);
    }
  }
  return r;
}

// 16-byte global load / store of eight elements.
CL_DEVICE u32x4 ld16(const elem_t* p) { return *reinterpret_cast<const u32x4*>(p); }
CL_DEVICE void st16(elem_t* p, u32x4 v) { *reinterpret_cast<u32x4*>(p) = v; }
CL_DEVICE elem8 as_elem8(u32x4 v) { return __builtin_bit_cast(elem8, v); }
CL_DEVICE u32x4 as_u32x4(elem8 v) { return __builtin_bit_cast(u32x4, v); }

// In-register 8x8 transpose of 16-bit elements.  in[e] holds row e (eight columns); out[j]
// receives column j (eight rows).  Row-major global tensors hand a lane eight neighbours of
// the *minor* axis per 16-byte load, while a matrix-core operand wants eight neighbours of
// the contraction axis: this turns one into the other without touching LDS (32 byte-permutes).
CL_DEVICE void transpose8x8(const u32x4 (&in)[8], u32x4 (&out)[8]) {
#pragma unroll
  for (int q = 0; q < 4; ++q) {      // column pair (2q, 2q+1) lives in dword q of every row
#pragma unroll
    for (int p = 0; p < 4; ++p) {    // row pair (2p, 2p+1) becomes dword p of the output
      // one byte-permute each: bytes 0-3 of the selector's source pair are x, bytes 4-7 are y
      u32 x = in[2 * p][q], y = in[2 * p + 1][q];
      out[2 * q][p] = __builtin_amdgcn_perm(y, x, 0x05040100u);      // (x & 0xffff) | (y << 16)
      out[2 * q + 1][p] = __builtin_amdgcn_perm(y, x, 0x07060302u);  // (x >> 16) | (y & 0xffff0000)
    }
  }
}

CL_DEVICE elem_t to_elem(float x) { return (elem_t)x; }
CL_DEVICE float to_f32(elem_t x) { return (float)x; }
