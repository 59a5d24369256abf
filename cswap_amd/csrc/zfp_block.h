// zfp_block.h -- one 4x4x4 fp32 block of the ZFP fixed-rate codec, written so
// that ONE LANE codes ONE BLOCK entirely in registers.
//
// The same source compiles for the device (hipcc) and for the host (any C++17
// compiler), so the block logic can be checked on a CPU before it ever runs on
// a GPU.  Nothing here touches memory except through the Mem object (or32 / ld32
// on a bit region) the caller passes in.
//
// What it implements (reference: the cuZFP snapshot of zfp 0.5.5 in
// CSWAP+/zfp): block-floating-point cast (encode.cuh:40-71,120-149), the
// decorrelating lifting transform (encode.cuh:73-99,154-175; inverse
// shared.h:217-248, decode.cuh:184-201), negabinary + sequency reorder
// (encode.cuh:203-212, constants.h:8-93) and the embedded bit-plane coder
// (encode.cuh:306-345; decoder decode.cuh:127-179).
//
// How it differs from the reference's formulation (results are identical):
//  * The 64x32 bit matrix of coefficients is transposed once with a butterfly
//    network instead of extracting each plane bit by bit.
//  * The coder emits whole runs: "group test 1, t zeros, terminating 1" is two
//    single-bit ORs into a zeroed bit region, placed with a count-trailing-zeros,
//    not t+2 single-bit writes; nothing is accumulated or flushed.
//  * The bit budget is applied as a cut of the unconstrained code at maxbits
//    (the reference's per-bit budget counter stops the same sequence of writes
//    at the same place, so the kept prefix is the same).
//  * The low 16 bit planes are only transposed and coded when some block of the
//    wavefront still has budget left after the top 16.
#pragma once
#include <stdint.h>

#if defined(__HIPCC__)
#include <hip/hip_runtime.h>
#define CSWAP_HD __host__ __device__ __forceinline__
#else
#include <math.h>
#define CSWAP_HD inline
#endif

namespace cswap {

// ---------------------------------------------------------------- permutation
// Sequency order of the coefficients: PERM3[i] = x + 4y + 16z of the i-th
// coefficient, sorted by x+y+z, then x^2+y^2+z^2 (table data as in
// CSWAP+/zfp/constants.h:8-93).
#define CSWAP_P3(x, y, z) ((x) + 4 * ((y) + 4 * (z)))
#define CSWAP_PERM3_LIST                                                               \
  CSWAP_P3(0,0,0), CSWAP_P3(1,0,0), CSWAP_P3(0,1,0), CSWAP_P3(0,0,1), CSWAP_P3(0,1,1), \
  CSWAP_P3(1,0,1), CSWAP_P3(1,1,0), CSWAP_P3(2,0,0), CSWAP_P3(0,2,0), CSWAP_P3(0,0,2), \
  CSWAP_P3(1,1,1), CSWAP_P3(2,1,0), CSWAP_P3(2,0,1), CSWAP_P3(0,2,1), CSWAP_P3(1,2,0), \
  CSWAP_P3(1,0,2), CSWAP_P3(0,1,2), CSWAP_P3(3,0,0), CSWAP_P3(0,3,0), CSWAP_P3(0,0,3), \
  CSWAP_P3(2,1,1), CSWAP_P3(1,2,1), CSWAP_P3(1,1,2), CSWAP_P3(0,2,2), CSWAP_P3(2,0,2), \
  CSWAP_P3(2,2,0), CSWAP_P3(3,1,0), CSWAP_P3(3,0,1), CSWAP_P3(0,3,1), CSWAP_P3(1,3,0), \
  CSWAP_P3(1,0,3), CSWAP_P3(0,1,3), CSWAP_P3(1,2,2), CSWAP_P3(2,1,2), CSWAP_P3(2,2,1), \
  CSWAP_P3(3,1,1), CSWAP_P3(1,3,1), CSWAP_P3(1,1,3), CSWAP_P3(3,2,0), CSWAP_P3(3,0,2), \
  CSWAP_P3(0,3,2), CSWAP_P3(2,3,0), CSWAP_P3(2,0,3), CSWAP_P3(0,2,3), CSWAP_P3(2,2,2), \
  CSWAP_P3(3,2,1), CSWAP_P3(3,1,2), CSWAP_P3(1,3,2), CSWAP_P3(2,3,1), CSWAP_P3(2,1,3), \
  CSWAP_P3(1,2,3), CSWAP_P3(0,3,3), CSWAP_P3(3,0,3), CSWAP_P3(3,3,0), CSWAP_P3(3,2,2), \
  CSWAP_P3(2,3,2), CSWAP_P3(2,2,3), CSWAP_P3(1,3,3), CSWAP_P3(3,1,3), CSWAP_P3(3,3,1), \
  CSWAP_P3(2,3,3), CSWAP_P3(3,2,3), CSWAP_P3(3,3,2), CSWAP_P3(3,3,3)

struct Perm3 {
  int v[64];
};
constexpr Perm3 kPerm3 = {{CSWAP_PERM3_LIST}};

// ---------------------------------------------------------------- small helpers
constexpr uint32_t kNegabinary = 0xaaaaaaaau;
CSWAP_HD uint32_t int2nb(int32_t x) { return ((uint32_t)x + 0xaaaaaaaau) ^ 0xaaaaaaaau; }
CSWAP_HD int32_t nb2int(uint32_t u) { return (int32_t)((u ^ 0xaaaaaaaau) - 0xaaaaaaaau); }

CSWAP_HD int ctz64(uint64_t v)  // 64 for v == 0
{
#if defined(__HIP_DEVICE_COMPILE__)
  return v ? __builtin_ctzll(v) : 64;
#else
  return v ? __builtin_ctzll(v) : 64;
#endif
}

// count of trailing zeros of a 32-bit word; some value >= 32 for v == 0 (the
// device instruction gives 0xffffffff, which callers only compare and clamp)
CSWAP_HD unsigned ctz32_or_more(uint32_t v)
{
#if defined(__HIP_DEVICE_COMPILE__)
  unsigned t;
  asm("v_ffbl_b32 %0, %1" : "=v"(t) : "v"(v));
  return t;
#else
  return v ? (unsigned)__builtin_ctz(v) : 0xffffffffu;
#endif
}

CSWAP_HD uint64_t low_mask(unsigned n)  // n in 0..64
{
  return n >= 64 ? ~(uint64_t)0 : (((uint64_t)1 << n) - 1);
}

// Division of a 31-bit number by a fixed divisor d >= 1 as a multiply and a
// shift: with l = ceil(log2 d) and mul = ceil(2^(31+l) / d) (which fits 32 bits),
// floor(b / d) = (b * mul) >> (31 + l) for every b < 2^31 (Granlund & Montgomery,
// "Division by invariant integers using multiplication", theorem 4.2 with N = 31).
struct Div31 {
  uint32_t mul, shift;  // shift = 31 + l
};
inline Div31 make_div31(uint32_t d)
{
  uint32_t l = 0;
  while (((uint64_t)1 << l) < d) l++;
  Div31 r;
  r.mul = (uint32_t)((((uint64_t)1 << (31 + l)) + d - 1) / d);
  r.shift = 31 + l;
  return r;
}
CSWAP_HD uint32_t div31(uint32_t b, Div31 d) { return (uint32_t)(((uint64_t)b * d.mul) >> d.shift); }

CSWAP_HD unsigned sub_sat(unsigned a, unsigned b)  // max(a - b, 0)
{
#if defined(__HIP_DEVICE_COMPILE__)
  return __builtin_elementwise_sub_sat(a, b);
#else
  return a > b ? a - b : 0u;
#endif
}

CSWAP_HD float f32_from_bits(uint32_t b)
{
#if defined(__HIP_DEVICE_COMPILE__)
  return __uint_as_float(b);
#else
  union { uint32_t u; float f; } c; c.u = b; return c.f;
#endif
}
CSWAP_HD uint32_t f32_bits(float f)
{
#if defined(__HIP_DEVICE_COMPILE__)
  return __float_as_uint(f);
#else
  union { uint32_t u; float f; } c; c.f = f; return c.u;
#endif
}

// 2^e as a float for e in [-149, 127]; +inf above, 0 below (what ldexpf gives)
CSWAP_HD float pow2f(int e)
{
  if (e > 127) return f32_from_bits(0x7f800000u);
  if (e >= -126) return f32_from_bits((uint32_t)(e + 127) << 23);
  if (e >= -149) return f32_from_bits(1u << (e + 149));
  return 0.0f;
}

// 2^(e8 - 157) for the 8-bit exponent field e8 of a block header (0..255): the
// decoder's scale 2^(emax - 30) with emax = e8 - 127, as ldexpf(1, emax - 30)
// gives it: normal from e8 = 31, subnormal down to e8 = 8, zero below.
CSWAP_HD float decode_scale(uint32_t e8)
{
  uint32_t normal = (e8 - 30u) << 23;
  uint32_t sub = e8 >= 8u ? 1u << ((e8 - 8u) & 31u) : 0u;
  return f32_from_bits(e8 >= 31u ? normal : sub);
}

// ---------------------------------------------------------------- lifting
// wrap-around int32 arithmetic (as on the GPU the reference runs on)
CSWAP_HD int32_t wadd(int32_t a, int32_t b) { return (int32_t)((uint32_t)a + (uint32_t)b); }
CSWAP_HD int32_t wsub(int32_t a, int32_t b) { return (int32_t)((uint32_t)a - (uint32_t)b); }
CSWAP_HD int32_t wdbl(int32_t a) { return (int32_t)((uint32_t)a << 1); }

CSWAP_HD void fwd_lift4(int32_t& x, int32_t& y, int32_t& z, int32_t& w)
{
  x = wadd(x, w); x >>= 1; w = wsub(w, x);
  z = wadd(z, y); z >>= 1; y = wsub(y, z);
  x = wadd(x, z); x >>= 1; z = wsub(z, x);
  w = wadd(w, y); w >>= 1; y = wsub(y, w);
  w = wadd(w, y >> 1); y = wsub(y, w >> 1);
}

CSWAP_HD void inv_lift4(int32_t& x, int32_t& y, int32_t& z, int32_t& w)
{
  // The reference's steps of the form "a += b; b <<= 1; b -= a" (shared.h:241-245)
  // leave a' = a + b and b' = 2b - (a + b) = b - a: two operations in wrap-around
  // arithmetic instead of three.
  y = wadd(y, w >> 1); w = wsub(w, y >> 1);
  { int32_t y0 = y; y = wadd(y, w); w = wsub(w, y0); }
  { int32_t z0 = z; z = wadd(z, x); x = wsub(x, z0); }
  { int32_t y0 = y; y = wadd(y, z); z = wsub(z, y0); }
  { int32_t w0 = w; w = wadd(w, x); x = wsub(x, w0); }
}

// the same two functions on int64 coefficients (zfp_type_double / zfp_type_int64)
CSWAP_HD int64_t wadd(int64_t a, int64_t b) { return (int64_t)((uint64_t)a + (uint64_t)b); }
CSWAP_HD int64_t wsub(int64_t a, int64_t b) { return (int64_t)((uint64_t)a - (uint64_t)b); }

CSWAP_HD void fwd_lift4(int64_t& x, int64_t& y, int64_t& z, int64_t& w)
{
  x = wadd(x, w); x >>= 1; w = wsub(w, x);
  z = wadd(z, y); z >>= 1; y = wsub(y, z);
  x = wadd(x, z); x >>= 1; z = wsub(z, x);
  w = wadd(w, y); w >>= 1; y = wsub(y, w);
  w = wadd(w, y >> 1); y = wsub(y, w >> 1);
}

CSWAP_HD void inv_lift4(int64_t& x, int64_t& y, int64_t& z, int64_t& w)
{
  y = wadd(y, w >> 1); w = wsub(w, y >> 1);
  { int64_t y0 = y; y = wadd(y, w); w = wsub(w, y0); }
  { int64_t z0 = z; z = wadd(z, x); x = wsub(x, z0); }
  { int64_t y0 = y; y = wadd(y, z); z = wsub(z, y0); }
  { int64_t w0 = w; w = wadd(w, x); x = wsub(x, w0); }
}

// b[x + 4y + 16z]; forward order x, y, z; inverse z, y, x
template <class I>
CSWAP_HD void fwd_xform3(I (&b)[64])
{
#pragma unroll
  for (int i = 0; i < 16; i++) fwd_lift4(b[4 * i], b[4 * i + 1], b[4 * i + 2], b[4 * i + 3]);
#pragma unroll
  for (int z = 0; z < 4; z++)
#pragma unroll
    for (int x = 0; x < 4; x++)
      fwd_lift4(b[16 * z + x], b[16 * z + x + 4], b[16 * z + x + 8], b[16 * z + x + 12]);
#pragma unroll
  for (int i = 0; i < 16; i++) fwd_lift4(b[i], b[i + 16], b[i + 32], b[i + 48]);
}

template <class I>
CSWAP_HD void inv_xform3_zy(I (&b)[64])  // the z and y passes; the x pass is one inv_lift4 per row
{
#pragma unroll
  for (int i = 0; i < 16; i++) inv_lift4(b[i], b[i + 16], b[i + 32], b[i + 48]);
#pragma unroll
  for (int z = 0; z < 4; z++)
#pragma unroll
    for (int x = 0; x < 4; x++)
      inv_lift4(b[16 * z + x], b[16 * z + x + 4], b[16 * z + x + 8], b[16 * z + x + 12]);
}

template <class I>
CSWAP_HD void inv_xform3(I (&b)[64])
{
  inv_xform3_zy(b);
#pragma unroll
  for (int i = 0; i < 16; i++) inv_lift4(b[4 * i], b[4 * i + 1], b[4 * i + 2], b[4 * i + 3]);
}

// ---------------------------------------------------------------- bit transpose
// In-place transpose of a 32x32 bit matrix held as 32 words: afterwards bit i
// of a[k] is what bit k of a[i] was.  Five butterfly stages; stage J swaps the
// upper-right and lower-left JxJ sub-blocks of every 2Jx2J tile.  The stages
// commute (each exchanges one row-index bit with one column-index bit), and
// after stage 16 the rows 16..31 hold only the high 16 bit-columns of the input,
// so the top 16 planes can be finished without touching rows 0..15.
//
// On the device every output word of a stage is one instruction after at most
// one shift: a byte permute for J = 16 and 8, a three-input bitwise function for
// J = 4, 2, 1.  They are written as builtins because the generic and/or/shift
// form gets re-associated across stages into longer sequences.
//
// Negabinary (encode.cuh:203-212, shared.h:176-181) is u = (x + c) ^ c with
// c = 0xaaaaaaaa.  The xor with c complements the odd bit planes, and J = 1 is
// the stage that pairs plane 2j with plane 2j+1, so it can complement for free:
// kNotOut complements the odd rows it writes (values -> planes, J = 1 last),
// kNotIn complements the odd rows it reads (planes -> values, J = 1 first).
enum { kPlain = 0, kNotOut = 1, kNotIn = 2 };

CSWAP_HD uint32_t bit_select(uint32_t m, uint32_t a, uint32_t b)  // m ? a : b
{
#if defined(__HIP_DEVICE_COMPILE__)
  return __builtin_amdgcn_bitop3_b32(m, a, b, 0xca);
#else
  return (a & m) | (b & ~m);
#endif
}
CSWAP_HD uint32_t bit_select_nb(uint32_t m, uint32_t a, uint32_t b)  // m ? a : ~b
{
#if defined(__HIP_DEVICE_COMPILE__)
  return __builtin_amdgcn_bitop3_b32(m, a, b, 0xc5);
#else
  return (a & m) | (~b & ~m);
#endif
}
CSWAP_HD uint32_t bit_select_nn(uint32_t m, uint32_t a, uint32_t b)  // ~(m ? a : b)
{
#if defined(__HIP_DEVICE_COMPILE__)
  return __builtin_amdgcn_bitop3_b32(m, a, b, 0x35);
#else
  return ~((a & m) | (b & ~m));
#endif
}

// A constant held in a vector register: the three-input bitwise instruction issues
// at twice the rate when none of its operands is a scalar register.
template <uint32_t C>
CSWAP_HD uint32_t vector_const()
{
#if defined(__HIP_DEVICE_COMPILE__)
  uint32_t v;
  asm("v_mov_b32 %0, %1" : "=v"(v) : "i"(C));
  return v;
#else
  return C;
#endif
}

// VM: the stage's mask in a vector register (one more register while the stage runs)
template <int J, int R0, int R1, int NB = kPlain, bool VM = false>
CSWAP_HD void tr_stage(uint32_t (&a)[32])
{
  static_assert(NB == kPlain || J == 1, "only the stage that pairs neighbouring planes can complement them");
  constexpr uint32_t mc = J == 16 ? 0x0000ffffu : J == 8 ? 0x00ff00ffu : J == 4 ? 0x0f0f0f0fu
                          : J == 2 ? 0x33333333u : 0x55555555u;
  const uint32_t m = VM && J <= 4 ? vector_const<mc>() : mc;
#pragma unroll
  for (int r = R0; r < R1; r++) {
    if (r & J) continue;
    const uint32_t lo = a[r], hi = a[r + J];
#if defined(__HIP_DEVICE_COMPILE__)
    if (J == 16) {  // bytes, low to high: lo0 lo1 hi0 hi1 / lo2 lo3 hi2 hi3
      a[r] = __builtin_amdgcn_perm(hi, lo, 0x05040100u);
      a[r + J] = __builtin_amdgcn_perm(hi, lo, 0x07060302u);
      continue;
    }
    if (J == 8) {  // lo0 hi0 lo2 hi2 / lo1 hi1 lo3 hi3
      a[r] = __builtin_amdgcn_perm(hi, lo, 0x06020400u);
      a[r + J] = __builtin_amdgcn_perm(hi, lo, 0x07030501u);
      continue;
    }
#endif
    if (NB == kNotIn) {  // hi is an odd plane: use its complement (the bit shifted in lands where m selects lo)
      a[r] = bit_select_nb(m, lo, hi << J);
      a[r + J] = bit_select_nb(m, lo >> J, hi);
    } else if (NB == kNotOut) {  // a[r + J] is an odd plane: store its complement
      a[r] = bit_select(m, lo, hi << J);
      a[r + J] = bit_select_nn(m, lo >> J, hi);
    } else {
      a[r] = bit_select(m, lo, hi << J);
      a[r + J] = bit_select(m, lo >> J, hi);
    }
  }
}

// stages 8,4,2,1 on rows [R0, R0+16); with kNotIn the order is 1,2,4,8
template <int R0, int NB = kPlain>
CSWAP_HD void tr_half(uint32_t (&a)[32])
{
  if (NB == kNotIn) {
    tr_stage<1, R0, R0 + 16, kNotIn>(a);
    tr_stage<2, R0, R0 + 16>(a);
    tr_stage<4, R0, R0 + 16>(a);
    tr_stage<8, R0, R0 + 16>(a);
  } else {
    tr_stage<8, R0, R0 + 16>(a);
    tr_stage<4, R0, R0 + 16>(a);
    tr_stage<2, R0, R0 + 16>(a);
    tr_stage<1, R0, R0 + 16, NB>(a);
  }
}

CSWAP_HD void transpose32(uint32_t (&a)[32])
{
  tr_stage<16, 0, 32>(a);
  tr_half<16>(a);
  tr_half<0>(a);
}

// ---------------------------------------------------------------- block cast
// Biased exponent field of the largest magnitude in the block; 0 only for an
// all-zero block.  The reference's emax (encode.cuh:40-71) is E - 126 for a
// non-zero block (subnormals clamp to -126, which is E = 0) and -127 for a zero
// block, so the 8-bit header exponent e = emax + 127 is E + 1, or 0.
CSWAP_HD uint32_t block_header_e(const float (&f)[64])
{
  float m = 0.0f;
#pragma unroll
  for (int i = 0; i < 64; i++) m = fmaxf(m, fabsf(f[i]));
  uint32_t b = f32_bits(m);
  return b ? (b >> 23) + 1 : 0;
}

// "does any block of this wavefront still ..." -- on the host a block is alone
#if defined(__HIP_DEVICE_COMPILE__)
#define CSWAP_ANY(pred) (__builtin_amdgcn_ballot_w64(pred) != 0)
#else
#define CSWAP_ANY(pred) (pred)
#endif

// bit position -> byte offset of the dword that holds it.  On the device the two
// instructions are opaque to the compiler: a right shift and an and, both of which
// issue at twice the rate of the shift-left (or shift-left-and-add) that it would
// otherwise make of "dword index times four".
CSWAP_HD unsigned dword_of(unsigned bitpos)
{
#if defined(__HIP_DEVICE_COMPILE__)
  unsigned d;
  asm("v_lshrrev_b32 %0, 3, %1\n\tv_and_b32 %0, -4, %0" : "=v"(d) : "v"(bitpos));
  return d;
#else
  return (bitpos >> 3) & ~3u;
#endif
}

// Makes the compiler finish computing v at this point instead of sinking part of
// it into a later branch (used where one LDS round trip should cover two uses).
CSWAP_HD void settle(uint64_t& v)
{
#if defined(__HIP_DEVICE_COMPILE__)
  asm volatile("" : "+v"(v));
#else
  (void)v;
#endif
}

CSWAP_HD void settle32(unsigned& v)
{
#if defined(__HIP_DEVICE_COMPILE__)
  asm volatile("" : "+v"(v));
#else
  (void)v;
#endif
}

// Makes the compiler finish computing rows R0 .. R0+15 at this point of the
// instruction stream.  Left alone it postpones whichever half of a butterfly
// stage's results is needed later and keeps the stage's inputs in registers
// until then, next to the results already made.
template <int R0>
CSWAP_HD void settle16(uint32_t (&a)[32])
{
#if defined(__HIP_DEVICE_COMPILE__)
  asm volatile("" : "+v"(a[R0 + 0]), "+v"(a[R0 + 1]), "+v"(a[R0 + 2]), "+v"(a[R0 + 3]), "+v"(a[R0 + 4]),
                    "+v"(a[R0 + 5]), "+v"(a[R0 + 6]), "+v"(a[R0 + 7]), "+v"(a[R0 + 8]), "+v"(a[R0 + 9]),
                    "+v"(a[R0 + 10]), "+v"(a[R0 + 11]), "+v"(a[R0 + 12]), "+v"(a[R0 + 13]), "+v"(a[R0 + 14]),
                    "+v"(a[R0 + 15]));
#else
  (void)a;
#endif
}

CSWAP_HD uint32_t funnel_shr(uint32_t hi, uint32_t lo, unsigned s)  // ({hi,lo} >> (s & 31)) low word
{
#if defined(__HIP_DEVICE_COMPILE__)
  return __builtin_amdgcn_alignbit(hi, lo, s);
#else
  s &= 31;
  return s ? (lo >> s) | (hi << (32 - s)) : lo;
#endif
}

// ---------------------------------------------------------------- encoder
// The block's bits are OR-ed into a zero-initialised bit region through
// mem.or32(byte_offset_of_a_dword, value); bit positions are absolute within that region.
// The block owns [pos0, pos0 + maxbits).  GUARD = true cuts every write at the
// end of the block (needed when the next block's bits follow immediately);
// GUARD = false lets the last plane spill up to 128 bits past the end, which the
// caller must provide as slack and ignore.
template <class Mem, bool GUARD, int SIZE = 64>
struct BlockEncoder {
  Mem& mem;
  unsigned pos, limit;
  unsigned n;  // coefficients already known significant

  CSWAP_HD BlockEncoder(Mem& m, unsigned pos0, unsigned maxbits) : mem(m), pos(pos0), limit(pos0 + maxbits), n(0) {}

  CSWAP_HD bool active() const { return pos < limit; }

  // append the low len (0..64) bits of v (bits at or above len must be 0); needs pos < limit
  CSWAP_HD void put(uint64_t v, unsigned len)
  {
    if (GUARD) {
      unsigned room = limit - pos;
      if (len > room) v &= low_mask(room);
    }
    unsigned d = dword_of(pos), s = pos & 31;
    uint64_t lo = v << s;
    uint32_t hi = ((uint32_t)(v >> 32) >> 1) >> (31 - s);
    mem.or32(d, (uint32_t)lo);
    mem.or32(d + 4, (uint32_t)(lo >> 32));
    mem.or32(d + 8, hi);
    pos += len;
  }

  CSWAP_HD void set_bit(unsigned b, bool on)
  {
    if (GUARD) on = on && b < limit;
    mem.or32(dword_of(b), on ? (1u << (b & 31)) : 0u);
  }

  // one bit plane: x bit i = this plane's bit of coefficient i (encode.cuh:331-344)
  CSWAP_HD void plane(uint64_t x)
  {
    if (!active()) return;
    // first n coefficients verbatim: x minus its part at and above bit n
    uint64_t rest = n < 64 ? x >> n : 0;
    put(n < 64 ? x ^ (rest << n) : x, n);
    if (n < SIZE) {
      bool more = true;
      // Without the guard a block that runs out of budget inside this loop simply goes
      // on to the end of the plane: what it writes past its end (less than 128 bits) lands
      // in the slack and is dropped.
      while (rest != 0 && more && (!GUARD || pos < limit)) {
        unsigned t1;  // zeros before the next one-bit, and that bit
        if (CSWAP_ANY((uint32_t)rest == 0)) t1 = (unsigned)ctz64(rest) + 1;
        else t1 = ctz32_or_more((uint32_t)rest) + 1;
        unsigned q = pos + t1;
        n += t1;
        more = n < SIZE;                     // a one-bit at the last position is implied, not written
        set_bit(pos, true);                  // positive group test
        set_bit(q, more);                    // the zeros, then the one-bit
        pos = q + (more ? 1u : 0u);
        rest >>= t1 & 63;                    // t1 = 64 only for the last coefficient: more is false, rest is not used again
      }
      // negative group test: a zero bit.  Without the guard a position past the end is
      // harmless (nothing is written there and the next plane sees the block as full)
      if (rest == 0 && n < SIZE && (!GUARD || pos < limit)) pos++;
    }
  }

  // One of the leading planes.  While no block of the wavefront has found a
  // significant coefficient and the plane is empty in all of them, the plane
  // costs every block one zero bit and nothing else.
  CSWAP_HD void leading_plane(uint64_t x)
  {
    if (!CSWAP_ANY(x != 0 || n != 0)) {
      if (active()) pos++;
      return;
    }
    plane(x);
  }

  // Advances the state over a plane that somebody else codes (a block shared by two
  // wavefronts): the same n and pos that plane(x) leaves behind, in closed form.  acc is
  // the OR of every plane so far (n is one more than the index of its highest one-bit).
  // A plane costs its n verbatim bits; for every one-bit at or above n a positive group
  // test, the zeros before it and the bit itself, which is n_new - n value bits and
  // popcount tests; and a negative test at the end -- unless the last coefficient was
  // reached, which also saves that coefficient's one-bit (encode.cuh:331-344).
  CSWAP_HD void skip_plane(uint64_t x, uint64_t& acc)
  {
    static_assert(SIZE == 64, "the closed form is written for blocks of 64 coefficients");
    const uint64_t rest = n < 64 ? x >> n : 0;
    acc |= x;
    const unsigned n_new = acc ? 64u - (unsigned)__builtin_clzll(acc) : 0u;
    const unsigned tests = (unsigned)__builtin_popcountll(rest);
    pos += n_new + tests + (n_new < 64 ? 1u : (n < 64 ? ~0u : 0u));
    n = n_new;
  }
};

// 32 bit planes of 64 coefficients.  lo / hi hold the 32-bit words of the
// coefficients 0..31 / 32..63 in coding order with the negabinary constant
// already added (the xor happens inside the transpose); planes below kmin are
// not coded.  Top 16 planes first; the low 16 are only transposed if some block
// of the wavefront still has bit budget left after them.
template <class Enc>
CSWAP_HD void encode_planes32(uint32_t (&lo)[32], uint32_t (&hi)[32], Enc& enc, unsigned kmin = 0)
{
  tr_stage<16, 0, 32>(lo);
  tr_stage<16, 0, 32>(hi);
  // The low 16 rows are only used if the low planes get coded.  Left alone, the
  // compiler postpones computing them until then and keeps all 64 inputs of this
  // stage in registers through the coding of the top planes; pinning the 32
  // results here lets the inputs go (32 registers less, one more wavefront per SIMD).
  settle16<0>(lo);
  settle16<0>(hi);
  tr_stage<8, 16, 32>(lo);
  tr_stage<8, 16, 32>(hi);
  settle16<16>(lo);
  settle16<16>(hi);
  tr_stage<4, 16, 32, kPlain, true>(lo);
  tr_stage<4, 16, 32, kPlain, true>(hi);
  settle16<16>(lo);
  settle16<16>(hi);
  tr_stage<2, 16, 32, kPlain, true>(lo);
  tr_stage<2, 16, 32, kPlain, true>(hi);
  settle16<16>(lo);
  settle16<16>(hi);
  tr_stage<1, 16, 32, kNotOut, true>(lo);
  tr_stage<1, 16, 32, kNotOut, true>(hi);
#pragma unroll
  for (int k = 31; k >= 28; k--) enc.leading_plane(((uint64_t)hi[k] << 32) | lo[k]);
#pragma unroll
  for (int k = 27; k >= 16; k--) enc.plane(((uint64_t)hi[k] << 32) | lo[k]);
  if (CSWAP_ANY(enc.active())) {
    tr_half<0, kNotOut>(lo);
    tr_half<0, kNotOut>(hi);
#pragma unroll
    for (int k = 15; k >= 0; k--)
      if ((unsigned)k >= kmin) enc.plane(((uint64_t)hi[k] << 32) | lo[k]);
  }
}

// Integer back end of a 4x4x4 block: transform, reorder, bit planes, coder
// (encode.cuh:306-345 with the callers at :347-380).  ib is overwritten.
template <class Enc>
CSWAP_HD void encode_ints3(int32_t (&ib)[64], Enc& enc)
{
  fwd_xform3(ib);

  uint32_t lo[32], hi[32];
#pragma unroll
  for (int i = 0; i < 32; i++) {  // negabinary: the add here, the xor inside the transpose
    lo[i] = (uint32_t)ib[kPerm3.v[i]] + kNegabinary;
    hi[i] = (uint32_t)ib[kPerm3.v[32 + i]] + kNegabinary;
  }
  encode_planes32(lo, hi, enc);
}

// The same with int64 coefficients: 64 planes, coded as the 32 planes of the
// high words followed by the 32 planes of the low words.
constexpr uint64_t kNegabinary64 = 0xaaaaaaaaaaaaaaaaull;
template <class Enc>
CSWAP_HD void encode_ints3(int64_t (&ib)[64], Enc& enc, unsigned kmin)
{
  fwd_xform3(ib);
#pragma unroll
  for (int i = 0; i < 64; i++) ib[i] = (int64_t)((uint64_t)ib[i] + kNegabinary64);

  uint32_t lo[32], hi[32];
#pragma unroll
  for (int i = 0; i < 32; i++) {
    lo[i] = (uint32_t)((uint64_t)ib[kPerm3.v[i]] >> 32);
    hi[i] = (uint32_t)((uint64_t)ib[kPerm3.v[32 + i]] >> 32);
  }
  encode_planes32(lo, hi, enc);
  if (CSWAP_ANY(enc.active())) {
#pragma unroll
    for (int i = 0; i < 32; i++) {
      lo[i] = (uint32_t)(uint64_t)ib[kPerm3.v[i]];
      hi[i] = (uint32_t)(uint64_t)ib[kPerm3.v[32 + i]];
    }
    encode_planes32(lo, hi, enc, kmin);
  }
}

// Full block encode: f[x + 4y + 16z] (already padded for partial blocks).
template <bool GUARD, class Mem>
CSWAP_HD void encode_block(const float (&f)[64], unsigned pos0, unsigned maxbits, Mem& mem)
{
  uint32_t e = block_header_e(f);
  if (e == 0) return;  // all-zero block: every bit stays 0 (encode.cuh:357-358)
  BlockEncoder<Mem, GUARD> enc(mem, pos0, maxbits);
  enc.put(2 * e + 1, 9);

  // block-floating-point cast: scale 2^(30-emax) as a float, truncate.  (A branch-free
  // form of this power of two costs the register allocator three spills at 96 registers.)
  float s = pow2f(30 - ((int)e - 127));
  int32_t ib[64];
#pragma unroll
  for (int i = 0; i < 64; i++) ib[i] = (int32_t)(s * f[i]);
  encode_ints3(ib, enc);
}

// int32 block (zfp_type_int32): no header, no cast, the whole budget for the
// coder (encode.cuh:371-380).  ib is overwritten.
template <bool GUARD, class Mem>
CSWAP_HD void encode_block_i32(int32_t (&ib)[64], unsigned pos0, unsigned maxbits, Mem& mem)
{
  BlockEncoder<Mem, GUARD> enc(mem, pos0, maxbits);
  encode_ints3(ib, enc);
}

// ---- 64-bit element types (zfp_type_double, zfp_type_int64; cuZFP.cu:401-423)
CSWAP_HD double f64_from_bits(uint64_t b)
{
#if defined(__HIP_DEVICE_COMPILE__)
  return __longlong_as_double((long long)b);
#else
  union { uint64_t u; double f; } c; c.u = b; return c.f;
#endif
}
CSWAP_HD uint64_t f64_bits(double f)
{
#if defined(__HIP_DEVICE_COMPILE__)
  return (uint64_t)__double_as_longlong(f);
#else
  union { uint64_t u; double f; } c; c.f = f; return c.u;
#endif
}

// 2^e as a double for any e: +inf above 1023, subnormal down to -1074, 0 below (ldexp(1.0, e))
CSWAP_HD double pow2d(int e)
{
  if (e > 1023) return f64_from_bits(0x7ff0000000000000ull);
  if (e >= -1022) return f64_from_bits((uint64_t)(e + 1023) << 52);
  if (e >= -1074) return f64_from_bits((uint64_t)1 << (e + 1074));
  return 0.0;
}

// double -> int64, truncating; saturates out of range and maps NaN to 0 (C leaves
// both undefined; the scale 2^(62-emax) overflows for blocks below 2^-961)
CSWAP_HD int64_t sat_i64(double v)
{
  if (!(v == v)) return 0;
  if (v >= 9223372036854775808.0) return INT64_MAX;
  if (v <= -9223372036854775808.0) return INT64_MIN;
  return (int64_t)v;
}

// header exponent of a block of SIZE doubles given as bit patterns: E + 1 with E
// the biased exponent field of the largest magnitude (emax = E - 1022, clamped at
// -1022 for subnormals, encode.cuh:40-71), or 0 for an all-zero block
template <int SIZE>
CSWAP_HD uint32_t block_header_e64(const uint64_t (&q)[SIZE])
{
  uint64_t m = 0;  // magnitudes of finite doubles order like their bit patterns
#pragma unroll
  for (int i = 0; i < SIZE; i++) {
    uint64_t a = q[i] & 0x7fffffffffffffffull;
    m = a > m ? a : m;
  }
  return m ? (uint32_t)(m >> 52) + 1 : 0;
}

// planes below this one are not coded for a block of doubles with header
// exponent e (encode.cuh:10-15: precision = min(64, emax + 1074 + 8), emax = e - 1023)
CSWAP_HD unsigned kmin_f64(uint32_t e)
{
  int maxprec = (int)e - 1023 + 1082;
  return maxprec >= 64 ? 0u : (unsigned)(64 - maxprec);
}

// q[x + 4y + 16z]: the (padded) block as 64-bit patterns of doubles, or of int64 when INT
template <bool GUARD, bool INT, class Mem>
CSWAP_HD void encode_block_w64(const uint64_t (&q)[64], unsigned pos0, unsigned maxbits, Mem& mem)
{
  BlockEncoder<Mem, GUARD> enc(mem, pos0, maxbits);
  int64_t ib[64];
  unsigned kmin = 0;
  if (INT) {
#pragma unroll
    for (int i = 0; i < 64; i++) ib[i] = (int64_t)q[i];
  } else {
    uint32_t e = block_header_e64<64>(q);
    if (e == 0) return;
    enc.put(2 * (uint64_t)e + 1, 12);
    kmin = kmin_f64(e);
    double s = pow2d(62 - ((int)e - 1023));
#pragma unroll
    for (int i = 0; i < 64; i++) ib[i] = sat_i64(s * f64_from_bits(q[i]));
  }
  encode_ints3(ib, enc, kmin);
}

// ---------------------------------------------------------------- one block, two wavefronts
// The "pair" form of the encoder, for fields that are too small to fill the chip with one
// lane per block: a block is shared by lane l of two wavefronts (halves 0 and 1 of a
// workgroup), each of which does half of every phase, so that twice as many wavefronts
// with half the serial work each are in flight.  The halves exchange data through an
// Exchange object (LDS and workgroup barriers on the device, shared arrays and a thread
// barrier in the host build that the CPU tests run).  Results are those of encode_block.
//
//  load      half 0 holds the z-slices 0 and 3 of the block (p, q), half 1 the slices 2 and 1
//  maximum   each half over its 32 values, exchanged                          (exchange 1)
//  cast, lifting along x and y of both slices: no exchange
//  lifting along z (fwd_lift4 on (x, y, z, w) = slices 0, 1, 2, 3): its first two lines pair
//            slice 0 with 3 and slice 2 with 1, which is what each half holds; the rest pairs
//            x with z and w with y, so half 0 sends w and gets z, half 1 the reverse
//                                                                              (exchange 2)
//            half 0 ends with the coefficients of z-index 0 and 2, half 1 with 1 and 3
//  reorder   half 0 needs the coefficients 0..31 in coding order, half 1 the others: 19 of
//            the 32 that a half holds stay (a register renaming), 13 change sides  (exchange 3)
//  planes    each half transposes its 32 coefficients: its 32 bits of every plane  (exchange 4)
//  coder     both halves walk all planes; half 0 codes the odd ones, half 1 the even ones, and
//            each steps over the other's planes in closed form (BlockEncoder::skip_plane).
//            Both OR into the same bit region, which therefore has to take ORs from two
//            wavefronts (LDS atomics do).
struct SeqOf {
  int v[64];
};
constexpr SeqOf make_seq_of()
{
  SeqOf s = {};
  for (int i = 0; i < 64; i++) s.v[kPerm3.v[i]] = i;
  return s;
}
constexpr SeqOf kSeqOf = make_seq_of();  // position in coding order of the coefficient x + 4y + 16z

// Slot r (0..31) of what a half holds after the z pass: r < 16 is its own slice register
// (z-index 0 for half 0, 1 for half 1), r >= 16 the one that came from the partner and
// was finished here (z-index 2 for half 0, 3 for half 1); r & 15 = x + 4y.
template <int H>
struct PairMap {
  static constexpr int natural(int r) { return (r & 15) + 16 * (H == 0 ? (r < 16 ? 0 : 2) : (r < 16 ? 1 : 3)); }
  static constexpr bool stays(int r) { return (kSeqOf.v[natural(r)] >> 5) == H; }
  static constexpr int row(int r) { return kSeqOf.v[natural(r)] & 31; }  // row of the 32-row array of whoever gets it
  static constexpr int sent_before(int r)
  {
    int j = 0;
    for (int q = 0; q < r; q++) j += stays(q) ? 0 : 1;
    return j;
  }
};
constexpr int kPairSent = PairMap<0>::sent_before(32);
static_assert(kPairSent == 13 && PairMap<1>::sent_before(32) == 13, "13 coefficients change sides in each direction");

CSWAP_HD float pair_max(const float (&p)[16], const float (&q)[16])
{
  float m = 0.0f;
#pragma unroll
  for (int i = 0; i < 16; i++) m = fmaxf(m, fmaxf(fabsf(p[i]), fabsf(q[i])));
  return m;
}

// cast, lifting along x and y of both slices, and the first two lines of the lifting along z
CSWAP_HD void pair_cast_xy_z1(float s, const float (&p)[16], const float (&q)[16], int32_t (&ip)[16], int32_t (&iq)[16])
{
#pragma unroll
  for (int i = 0; i < 16; i++) {
    ip[i] = (int32_t)(s * p[i]);
    iq[i] = (int32_t)(s * q[i]);
  }
#pragma unroll
  for (int y = 0; y < 4; y++) {
    fwd_lift4(ip[4 * y], ip[4 * y + 1], ip[4 * y + 2], ip[4 * y + 3]);
    fwd_lift4(iq[4 * y], iq[4 * y + 1], iq[4 * y + 2], iq[4 * y + 3]);
  }
#pragma unroll
  for (int x = 0; x < 4; x++) {
    fwd_lift4(ip[x], ip[x + 4], ip[x + 8], ip[x + 12]);
    fwd_lift4(iq[x], iq[x + 4], iq[x + 8], iq[x + 12]);
  }
#pragma unroll
  for (int i = 0; i < 16; i++) {  // half 0: x += w; x >>= 1; w -= x.  half 1: z += y; z >>= 1; y -= z.
    ip[i] = wadd(ip[i], iq[i]);
    ip[i] >>= 1;
    iq[i] = wsub(iq[i], ip[i]);
  }
}

// the rest of the lifting along z; c receives the half's 32 coefficients in PairMap order
template <int H>
CSWAP_HD void pair_z2(const int32_t (&ip)[16], const int32_t (&iq)[16], const int32_t (&got)[16], int32_t (&c)[32])
{
#pragma unroll
  for (int i = 0; i < 16; i++) {
    if (H == 0) {  // x = ip, z = got:  x += z; x >>= 1; z -= x
      int32_t x = wadd(ip[i], got[i]);
      x >>= 1;
      c[i] = x;
      c[16 + i] = wsub(got[i], x);
    } else {       // w = got, y = iq:  w += y; w >>= 1; y -= w; w += y >> 1; y -= w >> 1
      int32_t w = wadd(got[i], iq[i]);
      w >>= 1;
      int32_t y = wsub(iq[i], w);
      w = wadd(w, y >> 1);
      y = wsub(y, w >> 1);
      c[i] = y;
      c[16 + i] = w;
    }
  }
}

// the half's 32 bits of the planes 31..16: rows 16..31 of a afterwards (rows 0..15 keep what
// pair_low_planes needs)
CSWAP_HD void pair_top_planes(uint32_t (&a)[32])
{
  tr_stage<16, 0, 32>(a);
  settle16<0>(a);
  tr_stage<8, 16, 32>(a);
  settle16<16>(a);
  tr_stage<4, 16, 32, kPlain, true>(a);
  settle16<16>(a);
  tr_stage<2, 16, 32, kPlain, true>(a);
  settle16<16>(a);
  tr_stage<1, 16, 32, kNotOut, true>(a);
}
CSWAP_HD void pair_low_planes(uint32_t (&a)[32]) { tr_half<0, kNotOut>(a); }

// 16 planes, highest first (x[15] .. x[0]); half 0 codes the odd ones.  top: these are the
// planes 31..16, of which the first four get the treatment of leading planes.
template <int H, class Enc>
CSWAP_HD void pair_code16(const uint64_t (&x)[16], Enc& enc, uint64_t& acc, bool top)
{
#pragma unroll
  for (int k = 15; k >= 0; k--) {
    if (!CSWAP_ANY(enc.active())) continue;  // every block of the wavefront is out of budget: nothing more is written
    if ((k & 1) == (H == 0 ? 1 : 0)) {
      if (top && k >= 12) enc.leading_plane(x[k]);
      else enc.plane(x[k]);
      acc |= x[k];
    } else {
      enc.skip_plane(x[k], acc);
    }
  }
}

// One half's share of a block.  p, q: the half's two z-slices ([x + 4y]; half 0: z = 0 and 3,
// half 1: z = 2 and 1); live: false for the lanes past the end of the field (they go through
// every exchange and write nothing).  The block owns [pos0, pos0 + maxbits) of the zeroed bit
// region behind mem plus 128 bits of slack (unguarded coder).
//
// Exchange (every call is made by both halves, in this order):
//   float    other_max(float)                      my maximum out, the partner's back
//   void     swap16(const int32_t(&)[16], int32_t(&)[16])
//   void     seq_put(int slot, uint32_t), seq_sync(), uint32_t seq_get(int slot)
//   void     plane_put(int k, uint32_t), plane_sync(), uint64_t plane_get(int k)   (both halves' words)
//   bool     more(bool)                            half 0's answer for both; also orders the
//                                                  coder's writes before what follows
//   void     done()                                after the low planes, if more() said yes
template <int H, class Ex, class Mem>
CSWAP_HD void pair_encode_half(const float (&p)[16], const float (&q)[16], bool live, unsigned pos0, unsigned maxbits,
                               Mem& mem, Ex& ex)
{
  const float mine = pair_max(p, q);
  const uint32_t mb = f32_bits(fmaxf(mine, ex.other_max(mine)));
  const uint32_t e = (live && mb) ? (mb >> 23) + 1 : 0;  // as block_header_e
  const float s = e ? pow2f(30 - ((int)e - 127)) : 0.0f;

  int32_t ip[16], iq[16], got[16], c[32];
  pair_cast_xy_z1(s, p, q, ip, iq);
  ex.swap16(H == 0 ? iq : ip, got);
  pair_z2<H>(ip, iq, got, c);

  uint32_t a[32];
#pragma unroll
  for (int r = 0; r < 32; r++) {  // negabinary: the add here, the xor inside the transpose
    const uint32_t u = (uint32_t)c[r] + kNegabinary;
    if (PairMap<H>::stays(r)) a[PairMap<H>::row(r)] = u;
    else ex.seq_put(PairMap<H>::sent_before(r), u);
  }
  ex.seq_sync();
#pragma unroll
  for (int r = 0; r < 32; r++)
    if (!PairMap<1 - H>::stays(r)) a[PairMap<1 - H>::row(r)] = ex.seq_get(PairMap<1 - H>::sent_before(r));

  pair_top_planes(a);
#pragma unroll
  for (int k = 0; k < 16; k++) ex.plane_put(k, a[16 + k]);
  ex.plane_sync();
  uint64_t x[16];
#pragma unroll
  for (int k = 0; k < 16; k++) x[k] = ex.plane_get(k);

  BlockEncoder<Mem, false> enc(mem, pos0, maxbits);
  if (e == 0) {
    enc.pos = enc.limit;  // an all-zero block (encode.cuh:357-358) or a lane past the end: nothing is written
  } else if (H == 0) {
    enc.put(2 * e + 1, 9);
  } else {
    enc.pos += 9;
  }
  uint64_t acc = 0;
  pair_code16<H>(x, enc, acc, true);
  if (ex.more(CSWAP_ANY(enc.active()))) {
    pair_low_planes(a);
#pragma unroll
    for (int k = 0; k < 16; k++) ex.plane_put(k, a[k]);
    ex.plane_sync();
#pragma unroll
    for (int k = 0; k < 16; k++) x[k] = ex.plane_get(k);
    pair_code16<H>(x, enc, acc, false);
    ex.done();
  }
}

// ---------------------------------------------------------------- decoder
// mem.ld32(byte_offset_of_a_dword) reads the bit region; positions are absolute within it
// and the block owns [pos0, pos0 + maxbits).  Reads may run up to 128 bits past
// the end of the block (the values are never used).
// FENCED: the caller guarantees that the bit right after the block reads as one.
// A run of zeros that the bit budget cuts short then ends at that bit by itself,
// and the step loop does not have to clamp the run to the bits that are left.
template <class Mem, int SIZE = 64, bool FENCED = false>
struct BlockDecoder {
  Mem& mem;
  unsigned pos, limit;
  int nrem;  // SIZE - 1 - (coefficients already known significant): -1 once all of them are

  CSWAP_HD BlockDecoder(Mem& m, unsigned pos0, unsigned maxbits) : mem(m), pos(pos0), limit(pos0 + maxbits), nrem(SIZE - 1) {}

  CSWAP_HD bool active() const { return pos < limit; }

  CSWAP_HD uint64_t window(unsigned p) const  // 64 stream bits starting at bit p
  {
    unsigned d = dword_of(p);
    uint32_t w0 = mem.ld32(d), w1 = mem.ld32(d + 4), w2 = mem.ld32(d + 8);
    return ((uint64_t)funnel_shr(w2, w1, p) << 32) | funnel_shr(w1, w0, p);
  }

  // mirror of BlockEncoder::plane (decode.cuh:141-173).  Written without early
  // exits: a block that is out of budget reads zero verbatim bits and never
  // enters the step loop, and when every coefficient is already significant the
  // plane is one 64-bit read.  Every group test is read from a window that is
  // already in registers: the first one sits right behind the verbatim bits, the
  // one after a run right behind the run's terminating one-bit, so the step loop
  // turns once per positive test and not at all for a plane that adds nothing.
  //
  // A turn of the step loop looks at 32 stream bits.  That is enough when the run
  // ends, or the coefficients run out, within 30 bits (the next group test is then
  // inside the window as well); when some block of the wavefront needs more, the
  // turn is redone on 64 bits for all of them.
  CSWAP_HD uint64_t plane()
  {
    const unsigned n = (unsigned)(SIZE - 1 - nrem);
    unsigned left = sub_sat(limit, pos);
    unsigned m = n < left ? n : left;
    uint64_t w = window(pos);
    uint64_t above = w >> (m & 63);               // what follows the m verbatim bits (m = 64: not used)
    settle(above);                                // one shift serves the verbatim mask and the group test
    uint64_t x = w ^ (m < 64 ? above << m : 0);   // the low m bits of w
    pos += m;
    bool go = nrem >= 0 && pos < limit;           // a group test follows (then m = n < 64)
    bool test = go && ((uint32_t)above & 1u);
    pos += go ? 1u : 0u;
    if (test) {                                   // positive group test: a run of zeros, then a one
      unsigned d = dword_of(pos);
      uint32_t w0 = mem.ld32(d), w1 = mem.ld32(d + 4);
      do {
        uint32_t lo = funnel_shr(w1, w0, pos);
        unsigned maxrun = (unsigned)nrem;         // the run cannot pass the last coefficient
        if (!FENCED) {
          unsigned avail = limit - pos;
          maxrun = maxrun < avail ? maxrun : avail;
        }
        unsigned t = ctz32_or_more(lo);           // at least 32 when the window holds no one-bit
        unsigned r = t < maxrun ? t : maxrun;
        uint32_t after = lo >> (t & 31);          // bit 0: the one that ended the run, bit 1: the next group test
        if (CSWAP_ANY(r > 30)) {
          const uint32_t w2 = mem.ld32(d + 8);
          const uint64_t w64 = ((uint64_t)funnel_shr(w2, w1, pos) << 32) | lo;
          t = (unsigned)ctz64(w64);
          r = t < maxrun ? t : maxrun;
          after = (uint32_t)(w64 >> (t & 63));
        }
        // If there is another turn, it starts behind the one-bit and the group test
        // that follow these t zeros: its window is asked for now, so that the read
        // is under way while the rest of this turn is worked out.
        d = dword_of(pos + t + 2);
        w0 = mem.ld32(d);
        w1 = mem.ld32(d + 4);
        // found: t zeros, then a one; else the run reached the last position or the budget.
        // With the fence the run is only ever cut by the coefficients that are left, so
        // "found" is the same as "coefficients are left after this one": the carry of the
        // decrement below says it, and no comparison of its own is needed.
        unsigned left_after = (unsigned)nrem - r;
        x |= ((uint64_t)1 << (SIZE - 1)) >> left_after;
        unsigned dec;  // left_after - 1, written as an addition so that the carry is "some are left"
        const bool some_left = __builtin_uadd_overflow(left_after, 0xffffffffu, &dec);
        nrem = (int)dec;
        const bool found = FENCED ? some_left : t < maxrun;
        pos += r + (found ? 1u : 0u);   // FENCED and out of budget: "finds" the fence, pos = limit + 1
        settle32(pos);                  // (this sum and the one below are one add-with-carry each; merged they are four)
        // not found: the plane is over; found: t <= 62, so the next group test is bit 1 of `after`
        go = found && some_left && pos < limit;
        test = go && (after & 2u);
        pos += go ? 1u : 0u;
      } while (test);
    }
    return x;
  }

  // One of the leading planes.  While no block of the wavefront has a significant
  // coefficient, a plane that is empty in all of them is one zero bit per block
  // (mirror of BlockEncoder::leading_plane).
  CSWAP_HD uint64_t leading_plane()
  {
    if (!CSWAP_ANY(nrem != SIZE - 1)) {
      const bool act = pos < limit;
      const uint32_t bit = (mem.ld32(dword_of(pos)) >> (pos & 31)) & 1u;
      if (!CSWAP_ANY(act && bit)) {
        pos += act ? 1u : 0u;
        return 0;
      }
    }
    return plane();
  }
};

// Block decode in two parts, so that a caller can finish, convert and store one
// x-row at a time instead of holding 64 finished values:
//   decode_block_zy  everything up to and including the inverse lifting along z
//                    and y; leaves ib[x + 4y + 16z] and the scale w
//   decode_row       inverse lifting along x of one row and the cast to float
// An empty block gives ib = 0 and w = 0, i.e. +0.0 everywhere.

// 32 bit planes -> the 32-bit words of 64 coefficients (lo: 0..31, hi: 32..63 in
// coding order).  Negabinary: the xor happens inside the transpose, the
// subtraction of the returned constant is left to the caller.  When the low 16
// planes are all zero they are not transposed, so their complemented odd planes
// (0xaaaa in every value) are missing from the minuend as well.
template <class Dec>
CSWAP_HD uint32_t decode_planes32(Dec& dec, uint32_t (&lo)[32], uint32_t (&hi)[32])
{
#pragma unroll
  for (int k = 31; k >= 16; k--) {  // planes that no block of the wavefront can reach are zero without a read
    uint64_t x = 0;
    if (CSWAP_ANY(dec.active())) x = k >= 28 ? dec.leading_plane() : dec.plane();
    lo[k] = (uint32_t)x;
    hi[k] = (uint32_t)(x >> 32);
  }
  tr_half<16, kNotIn>(lo);
  tr_half<16, kNotIn>(hi);
  uint32_t c = kNegabinary;
  if (CSWAP_ANY(dec.active())) {
#pragma unroll
    for (int k = 15; k >= 0; k--) {
      uint64_t x = dec.plane();
      lo[k] = (uint32_t)x;
      hi[k] = (uint32_t)(x >> 32);
    }
    tr_half<0, kNotIn>(lo);
    tr_half<0, kNotIn>(hi);
  } else {
#pragma unroll
    for (int k = 0; k < 16; k++) lo[k] = hi[k] = 0;
    c = kNegabinary & 0xffff0000u;
  }
  tr_stage<16, 0, 32>(lo);
  tr_stage<16, 0, 32>(hi);
  return c;
}

// Integer back end of a 4x4x4 block up to and including the inverse lifting
// along z and y (decode.cuh:127-179 and the first two passes of :181-226).
// inv_lift4 on inputs that still carry the negabinary constant (X = x + c and so
// on, mod 2^32): only w has to be freed of it before its shift; y drops it in the
// three-input add that follows, z + x drops both at once and x - z never had it.
CSWAP_HD void inv_lift4_biased(int32_t& x, int32_t& y, int32_t& z, int32_t& w, uint32_t c)
{
  const uint32_t X = (uint32_t)x, Y = (uint32_t)y, Z = (uint32_t)z;
  w = (int32_t)((uint32_t)w - c);
  y = (int32_t)(Y + (uint32_t)(w >> 1) + (0u - c));
  w = wsub(w, y >> 1);
  z = (int32_t)(Z + X + (0u - 2u * c));
  x = (int32_t)(X - Z);
  { int32_t y0 = y; y = wadd(y, w); w = wsub(w, y0); }
  { int32_t y0 = y; y = wadd(y, z); z = wsub(z, y0); }
  { int32_t w0 = w; w = wadd(w, x); x = wsub(x, w0); }
}

// Issue priority of the wavefront from here on, against the other wavefronts of its SIMD
// (s_setprio; nothing on the host).
template <int P>
CSWAP_HD void issue_priority()
{
#if defined(__HIP_DEVICE_COMPILE__)
  __builtin_amdgcn_s_setprio(P);
#endif
}

// The caller runs the bit planes at the highest issue priority: that part is one dependent
// chain through LDS reads per block, and every slot it waits for is added to its length.  The
// lifting that follows is independent work that fills whatever slots are left, at the lowest.
template <class Dec>
CSWAP_HD void decode_ints3_zy(Dec& dec, int32_t (&ib)[64])
{
  uint32_t lo[32], hi[32];
  const uint32_t c = decode_planes32(dec, lo, hi);
  issue_priority<0>();
#pragma unroll
  for (int i = 0; i < 32; i++) {  // still with the negabinary constant added: the z pass takes it out
    ib[kPerm3.v[i]] = (int32_t)lo[i];
    ib[kPerm3.v[32 + i]] = (int32_t)hi[i];
  }
#pragma unroll
  for (int i = 0; i < 16; i++) inv_lift4_biased(ib[i], ib[i + 16], ib[i + 32], ib[i + 48], c);
#pragma unroll
  for (int z = 0; z < 4; z++)
#pragma unroll
    for (int x = 0; x < 4; x++)
      inv_lift4(ib[16 * z + x], ib[16 * z + x + 4], ib[16 * z + x + 8], ib[16 * z + x + 12]);
}

// int64 coefficients: the high words from the first 32 planes, the low words from
// the next 32 (skipped, with nothing to subtract for them, when no block of the
// wavefront has budget left); whole inverse transform
template <class Dec>
CSWAP_HD void decode_ints3(Dec& dec, int64_t (&ib)[64])
{
  uint32_t lo[32], hi[32];
  uint64_t c = (uint64_t)decode_planes32(dec, lo, hi) << 32;
#pragma unroll
  for (int i = 0; i < 32; i++) {
    ib[kPerm3.v[i]] = (int64_t)((uint64_t)lo[i] << 32);
    ib[kPerm3.v[32 + i]] = (int64_t)((uint64_t)hi[i] << 32);
  }
  if (CSWAP_ANY(dec.active())) {
    c |= decode_planes32(dec, lo, hi);
#pragma unroll
    for (int i = 0; i < 32; i++) {
      ib[kPerm3.v[i]] |= (int64_t)(uint64_t)lo[i];
      ib[kPerm3.v[32 + i]] |= (int64_t)(uint64_t)hi[i];
    }
  }
#pragma unroll
  for (int i = 0; i < 64; i++) ib[i] = (int64_t)((uint64_t)ib[i] - c);
  issue_priority<0>();  // as in decode_ints3_zy: the planes above went first, the lifting fills in
  inv_xform3(ib);
}

// q[x + 4y + 16z] receives the block as 64-bit patterns (doubles, or int64 when INT);
// an empty block of doubles gives +0.0 everywhere
template <bool INT, bool FENCED = false, class Mem>
CSWAP_HD void decode_block_w64(Mem& mem, unsigned pos0, unsigned maxbits, uint64_t (&q)[64])
{
  BlockDecoder<Mem, 64, FENCED> dec(mem, pos0, maxbits);
  int emax = 0;
  if (!INT) {
    uint32_t h = (uint32_t)dec.window(pos0);
    if (!(h & 1)) {
#pragma unroll
      for (int i = 0; i < 64; i++) q[i] = 0;
      return;
    }
    emax = (int)((h >> 1) & 0x7ff) - 1023;
    dec.pos = pos0 + 12;
  }
  int64_t ib[64];
  decode_ints3(dec, ib);
  if (INT) {
#pragma unroll
    for (int i = 0; i < 64; i++) q[i] = (uint64_t)ib[i];
  } else {
    const double w = pow2d(emax - 62);
#pragma unroll
    for (int i = 0; i < 64; i++) q[i] = f64_bits(w * (double)ib[i]);
  }
}

template <bool FENCED = false, class Mem>
CSWAP_HD void decode_block_zy(Mem& mem, unsigned pos0, unsigned maxbits, int32_t (&ib)[64], float& w)
{
  BlockDecoder<Mem, 64, FENCED> dec(mem, pos0, maxbits);
  uint32_t h = (uint32_t)dec.window(pos0);
  // An empty block (flag bit 0) takes the same path with its bit budget already
  // spent: every plane then reads as zero, the coefficients come out as zero and
  // the scale is zero, i.e. +0.0 everywhere, without a separate zero-fill of ib.
  const bool coded = (h & 1) != 0;
  dec.pos = coded ? pos0 + 9 : dec.limit;
  decode_ints3_zy(dec, ib);
  w = coded ? decode_scale((h >> 1) & 0xffu) : 0.0f;
}

// int32 block (zfp_type_int32): no header; finish each x-row with inv_lift4
template <bool FENCED = false, class Mem>
CSWAP_HD void decode_block_i32_zy(Mem& mem, unsigned pos0, unsigned maxbits, int32_t (&ib)[64])
{
  BlockDecoder<Mem, 64, FENCED> dec(mem, pos0, maxbits);
  decode_ints3_zy(dec, ib);
}

template <bool FENCED = false, class Mem>
CSWAP_HD void decode_block_i32(Mem& mem, unsigned pos0, unsigned maxbits, int32_t (&ib)[64])
{
  decode_block_i32_zy<FENCED>(mem, pos0, maxbits, ib);
#pragma unroll
  for (int row = 0; row < 16; row++) inv_lift4(ib[4 * row], ib[4 * row + 1], ib[4 * row + 2], ib[4 * row + 3]);
}

// row = y + 4z; f receives the four values of that x-row
CSWAP_HD void decode_row(int32_t (&ib)[64], int row, float w, float (&f)[4])
{
  inv_lift4(ib[4 * row], ib[4 * row + 1], ib[4 * row + 2], ib[4 * row + 3]);
#pragma unroll
  for (int x = 0; x < 4; x++) f[x] = w * (float)ib[4 * row + x];
}

// Full block decode into f[x + 4y + 16z]
template <bool FENCED = false, class Mem>
CSWAP_HD void decode_block(Mem& mem, unsigned pos0, unsigned maxbits, float (&f)[64])
{
  int32_t ib[64];
  float w;
  decode_block_zy<FENCED>(mem, pos0, maxbits, ib, w);
#pragma unroll
  for (int row = 0; row < 16; row++) {
    float r[4];
    decode_row(ib, row, w, r);
#pragma unroll
    for (int x = 0; x < 4; x++) f[4 * row + x] = r[x];
  }
}

// ---------------------------------------------------------------- one block, two wavefronts: decoding
// The pair form of the decoder.  Where a bit plane starts in a block's stream is only known once
// the planes before it are decoded, so the planes stay one chain per block: half 0 decodes them
// for all 64 blocks (lane per block, as the one-wavefront kernel does) while half 1 waits; what
// comes after -- the bit transposes, the reorder, the inverse lifting, the cast and the stores --
// is split as in pair_encode_half, mirrored:
//   planes    half 0 hands over the plane words; each half takes its 32 bits of every plane: the
//             coefficients 32 H .. 32 H + 31 in coding order after the transposes   (exchange 1;
//             once more for the low 16 planes, when some block of the 64 has budget left for them)
//   reorder   half 0 needs the coefficients of z-index 0 and 2, half 1 those of 1 and 3: 19 of a
//             half's 32 are among its own, 13 come from the partner                    (exchange 2)
//   lifting along z (inv_lift4 on (x, y, z, w) = z-index 0, 1, 2, 3): its first lines pair y with
//             w and z with x -- what each half holds --, the last two pair y with z and w with x:
//             half 0 sends z and gets w, half 1 the reverse                            (exchange 3)
//             half 0 ends with the slices z = 0 and 3, half 1 with 2 and 1, as the encoder's halves
//             start
//   lifting along y and x of both slices, cast: no exchange
// Results are those of decode_block.
//
// Exchange (every call is made by both halves, in this order):
//   void     plane_put(int k, uint64_t), scale_put(float)        half 0 only, before planes_sync
//   bool     planes_sync(bool)              half 0's answer (do the low planes follow) for both
//   uint32_t plane_get(int k)               my 32 bits of plane word k;  float scale_get()
//   void     consumed(), low_sync()         around half 0's decoding of the low planes, if they follow
//   void     seq_put(int slot, uint32_t), seq_sync(), uint32_t seq_get(int slot)
//   void     swap16(const int32_t(&)[16], int32_t(&)[16])
template <class Dec>
CSWAP_HD void pair_decode16(Dec& dec, uint64_t (&x)[16], bool top)
{
#pragma unroll
  for (int k = 15; k >= 0; k--) {
    x[k] = 0;  // planes that no block of the wavefront can reach are zero without a read
    if (CSWAP_ANY(dec.active())) x[k] = (top && k >= 12) ? dec.leading_plane() : dec.plane();
  }
}

// p, q receive the half's two z-slices ([x + 4y]; half 0: z = 0 and 3, half 1: z = 2 and 1).
// The block owns [pos0, pos0 + maxbits) of the bit region behind mem, followed by a fence of
// one-bits (only half 0 reads it).
template <int H, class Ex, class Mem>
CSWAP_HD void pair_decode_half(Mem& mem, unsigned pos0, unsigned maxbits, Ex& ex, float (&p)[16], float (&q)[16])
{
  BlockDecoder<Mem, 64, true> dec(mem, pos0, maxbits);
  uint64_t x[16];
  bool any = false;
  if (H == 0) {
    const uint32_t h = (uint32_t)dec.window(pos0);
    const bool coded = (h & 1) != 0;  // an empty block: its budget counts as spent, every plane reads as zero
    dec.pos = coded ? pos0 + 9 : dec.limit;
    pair_decode16(dec, x, true);
#pragma unroll
    for (int k = 0; k < 16; k++) ex.plane_put(k, x[k]);
    ex.scale_put(coded ? decode_scale((h >> 1) & 0xffu) : 0.0f);
    any = CSWAP_ANY(dec.active());
  }
  const bool low = ex.planes_sync(any);
  uint32_t a[32];
#pragma unroll
  for (int k = 0; k < 16; k++) a[16 + k] = ex.plane_get(k);
  const float w = ex.scale_get();
  tr_half<16, kNotIn>(a);
  uint32_t c = kNegabinary;
  if (low) {
    ex.consumed();
    if (H == 0) {
      pair_decode16(dec, x, false);
#pragma unroll
      for (int k = 0; k < 16; k++) ex.plane_put(k, x[k]);
    }
    ex.low_sync();
#pragma unroll
    for (int k = 0; k < 16; k++) a[k] = ex.plane_get(k);
    tr_half<0, kNotIn>(a);
  } else {  // no low planes: their complemented odd planes are missing from the minuend as well
#pragma unroll
    for (int k = 0; k < 16; k++) a[k] = 0;
    c = kNegabinary & 0xffff0000u;
  }
  tr_stage<16, 0, 32>(a);

  // a[i] is coefficient 32 H + i of the coding order with the negabinary constant still added
#pragma unroll
  for (int r = 0; r < 32; r++)  // what the partner needs of mine
    if (!PairMap<1 - H>::stays(r)) ex.seq_put(PairMap<1 - H>::sent_before(r), a[PairMap<1 - H>::row(r)] - c);
  ex.seq_sync();
  int32_t v[32];
#pragma unroll
  for (int r = 0; r < 32; r++)
    v[r] = (int32_t)(PairMap<H>::stays(r) ? a[PairMap<H>::row(r)] - c : ex.seq_get(PairMap<H>::sent_before(r)));

  // lifting along z.  Half 0 holds x = v[i], z = v[16 + i]; half 1 holds y = v[i], w = v[16 + i].
  int32_t keep[16], send[16], got[16];
#pragma unroll
  for (int i = 0; i < 16; i++) {
    if (H == 0) {  // z += x; x -= z_before
      const int32_t z0 = v[16 + i];
      send[i] = wadd(z0, v[i]);
      keep[i] = wsub(v[i], z0);
    } else {       // y += w >> 1; w -= y >> 1; y += w; w -= y_before
      int32_t y = wadd(v[i], v[16 + i] >> 1);
      int32_t ww = wsub(v[16 + i], y >> 1);
      keep[i] = wadd(y, ww);
      send[i] = wsub(ww, y);
    }
  }
  ex.swap16(send, got);
  int32_t ip[16], iq[16];
#pragma unroll
  for (int i = 0; i < 16; i++) {
    if (H == 0) {  // keep = x, got = w:  w += x; x -= w_before   -> slices 0 (x) and 3 (w)
      iq[i] = wadd(got[i], keep[i]);
      ip[i] = wsub(keep[i], got[i]);
    } else {       // keep = y, got = z:  y += z; z -= y_before   -> slices 2 (z) and 1 (y)
      iq[i] = wadd(keep[i], got[i]);
      ip[i] = wsub(got[i], keep[i]);
    }
  }
#pragma unroll
  for (int xx = 0; xx < 4; xx++) {
    inv_lift4(ip[xx], ip[xx + 4], ip[xx + 8], ip[xx + 12]);
    inv_lift4(iq[xx], iq[xx + 4], iq[xx + 8], iq[xx + 12]);
  }
#pragma unroll
  for (int y = 0; y < 4; y++) {
    inv_lift4(ip[4 * y], ip[4 * y + 1], ip[4 * y + 2], ip[4 * y + 3]);
    inv_lift4(iq[4 * y], iq[4 * y + 1], iq[4 * y + 2], iq[4 * y + 3]);
  }
#pragma unroll
  for (int i = 0; i < 16; i++) {
    p[i] = w * (float)ip[i];
    q[i] = w * (float)iq[i];
  }
}

// ---------------------------------------------------------------- 2-D and 1-D blocks
// Blocks of 4x4 = 16 and 4 values (CSWAP+/zfp/encode2.cuh, encode1.cuh,
// decode2.cuh, decode1.cuh): same cast and coder with 16 / 4 coefficients, lifting
// along x then y (encode.cuh:177-201; inverse y then x, decode.cuh:203-226),
// coefficient order perm_2 / identity (constants.h:95-133).  The bit planes are
// formed with the same 32x32 transpose on zero-padded rows.
#define CSWAP_P2(i, j) ((i) + 4 * (j))
struct Perm2 {
  int v[16];
};
constexpr Perm2 kPerm2 = {{CSWAP_P2(0,0), CSWAP_P2(1,0), CSWAP_P2(0,1), CSWAP_P2(1,1), CSWAP_P2(2,0), CSWAP_P2(0,2),
                           CSWAP_P2(2,1), CSWAP_P2(1,2), CSWAP_P2(3,0), CSWAP_P2(0,3), CSWAP_P2(2,2), CSWAP_P2(3,1),
                           CSWAP_P2(1,3), CSWAP_P2(3,2), CSWAP_P2(2,3), CSWAP_P2(3,3)}};

// INT: f holds the bit patterns of int32 values (zfp_type_int32: no header, no cast)
template <int DIMS, bool GUARD, bool INT = false, class Mem>
CSWAP_HD void encode_block_low(const float (&f)[16], unsigned pos0, unsigned maxbits, Mem& mem)
{
  constexpr int SIZE = DIMS == 2 ? 16 : 4;
  BlockEncoder<Mem, GUARD, SIZE> enc(mem, pos0, maxbits);
  int32_t ib[16];
  if (INT) {
#pragma unroll
    for (int i = 0; i < SIZE; i++) ib[i] = (int32_t)f32_bits(f[i]);
  } else {
    float m = 0.0f;
#pragma unroll
    for (int i = 0; i < SIZE; i++) m = fmaxf(m, fabsf(f[i]));
    uint32_t mb = f32_bits(m);
    uint32_t e = mb ? (mb >> 23) + 1 : 0;
    if (e == 0) return;
    enc.put(2 * e + 1, 9);
    float s = pow2f(30 - ((int)e - 127));
#pragma unroll
    for (int i = 0; i < SIZE; i++) ib[i] = (int32_t)(s * f[i]);
  }
  uint32_t a[32];
#pragma unroll
  for (int i = 0; i < 32; i++) a[i] = 0;
  if (DIMS == 2) {
#pragma unroll
    for (int y = 0; y < 4; y++) fwd_lift4(ib[4 * y], ib[4 * y + 1], ib[4 * y + 2], ib[4 * y + 3]);
#pragma unroll
    for (int x = 0; x < 4; x++) fwd_lift4(ib[x], ib[x + 4], ib[x + 8], ib[x + 12]);
#pragma unroll
    for (int i = 0; i < 16; i++) a[i] = int2nb(ib[kPerm2.v[i]]);
  } else {
    fwd_lift4(ib[0], ib[1], ib[2], ib[3]);
#pragma unroll
    for (int i = 0; i < 4; i++) a[i] = int2nb(ib[i]);
  }
  transpose32(a);
#pragma unroll
  for (int k = 31; k >= 0; k--) enc.plane((uint64_t)a[k]);
}

template <int DIMS, bool INT = false, class Mem>
CSWAP_HD void decode_block_low(Mem& mem, unsigned pos0, unsigned maxbits, float (&f)[16])
{
  constexpr int SIZE = DIMS == 2 ? 16 : 4;
  BlockDecoder<Mem, SIZE> dec(mem, pos0, maxbits);
  int emax = 0;
  if (!INT) {
    uint32_t h = (uint32_t)dec.window(pos0);
    if (!(h & 1)) {
#pragma unroll
      for (int i = 0; i < 16; i++) f[i] = 0.0f;
      return;
    }
    emax = (int)((h >> 1) & 0xff) - 127;
    dec.pos = pos0 + 9;
  }
  uint32_t a[32];
#pragma unroll
  for (int k = 31; k >= 0; k--) a[k] = (uint32_t)dec.plane();
  transpose32(a);
  int32_t ib[16];
  if (DIMS == 2) {
#pragma unroll
    for (int i = 0; i < 16; i++) ib[kPerm2.v[i]] = nb2int(a[i]);
#pragma unroll
    for (int x = 0; x < 4; x++) inv_lift4(ib[x], ib[x + 4], ib[x + 8], ib[x + 12]);
#pragma unroll
    for (int y = 0; y < 4; y++) inv_lift4(ib[4 * y], ib[4 * y + 1], ib[4 * y + 2], ib[4 * y + 3]);
  } else {
#pragma unroll
    for (int i = 0; i < 4; i++) ib[i] = nb2int(a[i]);
    inv_lift4(ib[0], ib[1], ib[2], ib[3]);
  }
  if (INT) {
#pragma unroll
    for (int i = 0; i < SIZE; i++) f[i] = f32_from_bits((uint32_t)ib[i]);
  } else {
    float w = pow2f(emax - 30);
#pragma unroll
    for (int i = 0; i < SIZE; i++) f[i] = w * (float)ib[i];
  }
#pragma unroll
  for (int i = SIZE; i < 16; i++) f[i] = 0.0f;
}

// The same for 64-bit element types: q holds 64-bit patterns (doubles, or int64
// when INT); 64 planes coded as the planes of the high words, then of the low words.
template <int DIMS, bool GUARD, bool INT, class Mem>
CSWAP_HD void encode_block_low_w64(const uint64_t (&q)[16], unsigned pos0, unsigned maxbits, Mem& mem)
{
  constexpr int SIZE = DIMS == 2 ? 16 : 4;
  BlockEncoder<Mem, GUARD, SIZE> enc(mem, pos0, maxbits);
  int64_t ib[16];
  unsigned kmin = 0;
  if (INT) {
#pragma unroll
    for (int i = 0; i < SIZE; i++) ib[i] = (int64_t)q[i];
  } else {
    uint64_t m = 0;
#pragma unroll
    for (int i = 0; i < SIZE; i++) {
      uint64_t a = q[i] & 0x7fffffffffffffffull;
      m = a > m ? a : m;
    }
    uint32_t e = m ? (uint32_t)(m >> 52) + 1 : 0;
    if (e == 0) return;
    enc.put(2 * (uint64_t)e + 1, 12);
    kmin = kmin_f64(e);
    double s = pow2d(62 - ((int)e - 1023));
#pragma unroll
    for (int i = 0; i < SIZE; i++) ib[i] = sat_i64(s * f64_from_bits(q[i]));
  }
  uint64_t u[16];
  if (DIMS == 2) {
#pragma unroll
    for (int y = 0; y < 4; y++) fwd_lift4(ib[4 * y], ib[4 * y + 1], ib[4 * y + 2], ib[4 * y + 3]);
#pragma unroll
    for (int x = 0; x < 4; x++) fwd_lift4(ib[x], ib[x + 4], ib[x + 8], ib[x + 12]);
#pragma unroll
    for (int i = 0; i < 16; i++) u[i] = ((uint64_t)ib[kPerm2.v[i]] + kNegabinary64) ^ kNegabinary64;
  } else {
    fwd_lift4(ib[0], ib[1], ib[2], ib[3]);
#pragma unroll
    for (int i = 0; i < 4; i++) u[i] = ((uint64_t)ib[i] + kNegabinary64) ^ kNegabinary64;
  }
  uint32_t a[32];
#pragma unroll
  for (int i = 0; i < 32; i++) a[i] = i < SIZE ? (uint32_t)(u[i < SIZE ? i : 0] >> 32) : 0u;
  transpose32(a);
#pragma unroll
  for (int k = 31; k >= 0; k--) enc.plane((uint64_t)a[k]);
#pragma unroll
  for (int i = 0; i < 32; i++) a[i] = i < SIZE ? (uint32_t)u[i < SIZE ? i : 0] : 0u;
  transpose32(a);
#pragma unroll
  for (int k = 31; k >= 0; k--)
    if ((unsigned)k >= kmin) enc.plane((uint64_t)a[k]);
}

template <int DIMS, bool INT, class Mem>
CSWAP_HD void decode_block_low_w64(Mem& mem, unsigned pos0, unsigned maxbits, uint64_t (&q)[16])
{
  constexpr int SIZE = DIMS == 2 ? 16 : 4;
  BlockDecoder<Mem, SIZE> dec(mem, pos0, maxbits);
  int emax = 0;
#pragma unroll
  for (int i = 0; i < 16; i++) q[i] = 0;
  if (!INT) {
    uint32_t h = (uint32_t)dec.window(pos0);
    if (!(h & 1)) return;
    emax = (int)((h >> 1) & 0x7ff) - 1023;
    dec.pos = pos0 + 12;
  }
  uint32_t a[32];
  uint64_t u[16];
#pragma unroll
  for (int k = 31; k >= 0; k--) a[k] = (uint32_t)dec.plane();
  transpose32(a);
#pragma unroll
  for (int i = 0; i < SIZE; i++) u[i] = (uint64_t)a[i] << 32;
#pragma unroll
  for (int k = 31; k >= 0; k--) a[k] = (uint32_t)dec.plane();
  transpose32(a);
#pragma unroll
  for (int i = 0; i < SIZE; i++) u[i] |= a[i];
  int64_t ib[16];
  if (DIMS == 2) {
#pragma unroll
    for (int i = 0; i < 16; i++) ib[kPerm2.v[i]] = (int64_t)((u[i] ^ kNegabinary64) - kNegabinary64);
#pragma unroll
    for (int x = 0; x < 4; x++) inv_lift4(ib[x], ib[x + 4], ib[x + 8], ib[x + 12]);
#pragma unroll
    for (int y = 0; y < 4; y++) inv_lift4(ib[4 * y], ib[4 * y + 1], ib[4 * y + 2], ib[4 * y + 3]);
  } else {
#pragma unroll
    for (int i = 0; i < 4; i++) ib[i] = (int64_t)((u[i] ^ kNegabinary64) - kNegabinary64);
    inv_lift4(ib[0], ib[1], ib[2], ib[3]);
  }
  if (INT) {
#pragma unroll
    for (int i = 0; i < SIZE; i++) q[i] = (uint64_t)ib[i];
  } else {
    const double w = pow2d(emax - 62);
#pragma unroll
    for (int i = 0; i < SIZE; i++) q[i] = f64_bits(w * (double)ib[i]);
  }
}

// ---------------------------------------------------------------- partial blocks
// Padding rule for a 4-vector of which the first n entries are valid
// (encode.cuh:17-38): n=1 -> (a,a,a,a), n=2 -> (a,b,b,a), n=3 -> (a,b,c,a).
template <class T>
CSWAP_HD void pad4(T& a, T& b, T& c, T& d, unsigned n)
{
  if (n == 0) a = T(0);
  if (n <= 1) b = a;
  if (n <= 2) c = b;
  if (n <= 3) d = a;
}

template <class T>
CSWAP_HD void pad_block3(T (&f)[64], unsigned bx, unsigned by, unsigned bz)
{
#pragma unroll
  for (int z = 0; z < 4; z++) {
#pragma unroll
    for (int y = 0; y < 4; y++) {
      int o = 16 * z + 4 * y;
      pad4(f[o], f[o + 1], f[o + 2], f[o + 3], bx);
    }
#pragma unroll
    for (int x = 0; x < 4; x++) {
      int o = 16 * z + x;
      pad4(f[o], f[o + 4], f[o + 8], f[o + 12], by);
    }
  }
#pragma unroll
  for (int i = 0; i < 16; i++) pad4(f[i], f[i + 16], f[i + 32], f[i + 48], bz);
}

}  // namespace cswap
