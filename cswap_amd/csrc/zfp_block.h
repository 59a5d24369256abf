// zfp_block.h -- one 4x4x4 fp32 block of the ZFP fixed-rate codec, written so
// that ONE LANE codes ONE BLOCK entirely in registers.
//
// The same source compiles for the device (hipcc) and for the host (any C++17
// compiler), so the block logic can be checked on a CPU before it ever runs on
// a GPU.  Nothing here touches memory except through the Sink/Source objects
// the caller passes in.
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
//  * The coder emits whole runs: "group test 1, t zeros, terminating 1" is one
//    64-bit append found with a count-trailing-zeros, not t+2 single-bit writes.
//  * The bit budget is applied as a cut of the unconstrained code at maxbits
//    (the reference's per-bit budget counter stops the same sequence of writes
//    at the same place, so the kept prefix is the same).
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

CSWAP_HD uint64_t low_mask(unsigned n)  // n in 0..64
{
  return n >= 64 ? ~(uint64_t)0 : (((uint64_t)1 << n) - 1);
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
  y = wadd(y, w >> 1); w = wsub(w, y >> 1);
  y = wadd(y, w); w = wdbl(w); w = wsub(w, y);
  z = wadd(z, x); x = wdbl(x); x = wsub(x, z);
  y = wadd(y, z); z = wdbl(z); z = wsub(z, y);
  w = wadd(w, x); x = wdbl(x); x = wsub(x, w);
}

// b[x + 4y + 16z]; forward order x, y, z; inverse z, y, x
CSWAP_HD void fwd_xform3(int32_t (&b)[64])
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

CSWAP_HD void inv_xform3(int32_t (&b)[64])
{
#pragma unroll
  for (int i = 0; i < 16; i++) inv_lift4(b[i], b[i + 16], b[i + 32], b[i + 48]);
#pragma unroll
  for (int z = 0; z < 4; z++)
#pragma unroll
    for (int x = 0; x < 4; x++)
      inv_lift4(b[16 * z + x], b[16 * z + x + 4], b[16 * z + x + 8], b[16 * z + x + 12]);
#pragma unroll
  for (int i = 0; i < 16; i++) inv_lift4(b[4 * i], b[4 * i + 1], b[4 * i + 2], b[4 * i + 3]);
}

// ---------------------------------------------------------------- bit transpose
// In-place transpose of a 32x32 bit matrix held as 32 words: afterwards bit i
// of a[k] is what bit k of a[i] was.  Five butterfly stages; each swaps the
// upper-right and lower-left sub-blocks of every 2j x 2j tile.
template <int J>
CSWAP_HD void tr_stage(uint32_t (&a)[32])
{
  constexpr uint32_t m = J == 16 ? 0x0000ffffu : J == 8 ? 0x00ff00ffu : J == 4 ? 0x0f0f0f0fu
                         : J == 2 ? 0x33333333u : 0x55555555u;
#pragma unroll
  for (int r = 0; r < 32; r++) {
    if (r & J) continue;
    uint32_t lo = a[r], hi = a[r + J];
    a[r] = (lo & m) | ((hi << J) & ~m);
    a[r + J] = ((lo >> J) & m) | (hi & ~m);
  }
}

CSWAP_HD void transpose32(uint32_t (&a)[32])
{
  tr_stage<16>(a);
  tr_stage<8>(a);
  tr_stage<4>(a);
  tr_stage<2>(a);
  tr_stage<1>(a);
}

// ---------------------------------------------------------------- block cast
// Biased exponent field of the largest magnitude in the block; 0 only for an
// all-zero block.  The reference's emax (encode.cuh:40-71) is E - 126 for a
// non-zero block (subnormals clamp to -126, which is E = 0) and -127 for a zero
// block, so the 8-bit header exponent e = emax + 127 is E + 1, or 0.
CSWAP_HD uint32_t block_header_e(const float (&f)[64])
{
  uint32_t m = 0;  // |x| compares like its bit pattern
#pragma unroll
  for (int i = 0; i < 64; i++) {
    uint32_t a = f32_bits(f[i]) & 0x7fffffffu;
    m = a > m ? a : m;
  }
  return m ? (m >> 23) + 1 : 0;
}

// ---------------------------------------------------------------- encoder
// Appends bit strings to the block's own stream and hands out finished 64-bit
// words to the sink: sink.put(j, word) receives word j (bits 64j..64j+63 of
// the block); words at or past maxbits are dropped and the word that straddles
// maxbits is cut.
template <class Sink>
struct BitAppender {
  Sink& sink;
  uint64_t acc;
  unsigned accn;   // valid bits in acc, 0..63
  unsigned j;      // index of the word acc will become
  unsigned maxbits;

  CSWAP_HD BitAppender(Sink& s, unsigned mb) : sink(s), acc(0), accn(0), j(0), maxbits(mb) {}

  CSWAP_HD unsigned emitted() const { return 64 * j + accn; }
  CSWAP_HD bool full() const { return emitted() >= maxbits; }

  CSWAP_HD void out(uint64_t w)
  {
    unsigned base = 64 * j;
    if (base < maxbits) {
      unsigned room = maxbits - base;
      if (room < 64) w &= low_mask(room);
      sink.put(j, w);
    }
    j++;
  }

  // append the low len (0..64) bits of v; bits of v at or above len must be 0
  CSWAP_HD void put(uint64_t v, unsigned len)
  {
    acc |= v << accn;
    unsigned tot = accn + len;
    if (tot >= 64) {
      out(acc);
      unsigned used = 64 - accn;              // 1..64 bits of v went out
      acc = used >= 64 ? 0 : (v >> used);
      tot -= 64;
    }
    accn = tot;
  }

  CSWAP_HD void finish()
  {
    if (accn) { out(acc); acc = 0; accn = 0; }
  }
};

// Code the 32 bit planes x[31]..x[0] (x[k] bit i = bit k of coefficient i) into
// the appender until the block's bit budget is used up.
template <class Sink>
CSWAP_HD void encode_planes(BitAppender<Sink>& bs, const uint32_t (&plo)[32], const uint32_t (&phi)[32])
{
  unsigned n = 0;  // coefficients already known significant
#pragma unroll
  for (int k = 31; k >= 0; k--) {
    if (bs.full()) break;
    uint64_t x = ((uint64_t)phi[k] << 32) | plo[k];
    // first n coefficients: verbatim
    bs.put(x & low_mask(n), n);
    if (n < 64) {
      uint64_t rest = x >> n;
      for (;;) {
        if (rest == 0) { bs.put(0, 1); break; }       // negative group test
        unsigned t = (unsigned)ctz64(rest);            // zeros before the next one-bit
        bool last = (n + t == 63);                     // one-bit at position 63 is implied
        uint64_t v = last ? (uint64_t)1 : ((uint64_t)1 | ((uint64_t)2 << t));
        bs.put(v, t + (last ? 1u : 2u));               // test '1', t zeros, then '1'
        n += t + 1;
        rest = (rest >> t) >> 1;
        if (n >= 64 || bs.full()) break;
      }
    }
  }
}

// Full block encode: f[x + 4y + 16z] (already padded for partial blocks).
template <class Sink>
CSWAP_HD void encode_block(const float (&f)[64], unsigned maxbits, Sink& sink)
{
  uint32_t e = block_header_e(f);
  if (e == 0) return;  // all-zero block: every bit stays 0 (encode.cuh:357-358)
  BitAppender<Sink> bs(sink, maxbits);
  bs.put(2 * e + 1, 9);

  // block-floating-point cast: scale 2^(30-emax) as a float, truncate
  float s = pow2f(30 - ((int)e - 127));
  int32_t ib[64];
#pragma unroll
  for (int i = 0; i < 64; i++) ib[i] = (int32_t)(s * f[i]);

  fwd_xform3(ib);

  uint32_t lo[32], hi[32];
#pragma unroll
  for (int i = 0; i < 32; i++) {
    lo[i] = int2nb(ib[kPerm3.v[i]]);
    hi[i] = int2nb(ib[kPerm3.v[32 + i]]);
  }
  transpose32(lo);
  transpose32(hi);

  encode_planes(bs, lo, hi);
  bs.finish();
}

// ---------------------------------------------------------------- decoder
// Source: src.window(pos) returns the 64 stream bits of this block starting at
// block-relative bit position pos (bits past the end of the stream may be
// anything; they are never used).
template <class Source>
CSWAP_HD void decode_planes(Source& src, unsigned maxbits, uint32_t (&plo)[32], uint32_t (&phi)[32])
{
  unsigned pos = 9;
  unsigned n = 0;
#pragma unroll
  for (int k = 31; k >= 0; k--) {
    uint64_t x = 0;
    if (pos < maxbits) {
      unsigned left = maxbits - pos;
      unsigned m = n < left ? n : left;
      if (m) {
        x = src.window(pos) & low_mask(m);
        pos += m;
      }
      while (n < 64 && pos < maxbits) {
        uint64_t w = src.window(pos);
        pos++;
        if (!(w & 1)) break;                       // negative group test: plane done
        w >>= 1;                                   // 63 valid bits
        unsigned avail = maxbits - pos;
        unsigned maxrun = 63 - n < avail ? 63 - n : avail;
        unsigned t = (unsigned)ctz64(w);
        if (t < maxrun) { pos += t + 1; n += t; }  // t zeros then a one
        else { pos += maxrun; n += maxrun; }       // ran into position 63 or the budget
        x |= (uint64_t)1 << n;
        n++;
      }
    }
    plo[k] = (uint32_t)x;
    phi[k] = (uint32_t)(x >> 32);
  }
}

// Full block decode into f[x + 4y + 16z]; an empty block gives +0.0 everywhere.
template <class Source>
CSWAP_HD void decode_block(Source& src, unsigned maxbits, float (&f)[64])
{
  uint64_t h = src.window(0);
  if (!(h & 1)) {
#pragma unroll
    for (int i = 0; i < 64; i++) f[i] = 0.0f;
    return;
  }
  int emax = (int)((h >> 1) & 0xff) - 127;

  uint32_t lo[32], hi[32];
  decode_planes(src, maxbits, lo, hi);
  transpose32(lo);
  transpose32(hi);

  int32_t ib[64];
#pragma unroll
  for (int i = 0; i < 32; i++) {
    ib[kPerm3.v[i]] = nb2int(lo[i]);
    ib[kPerm3.v[32 + i]] = nb2int(hi[i]);
  }
  inv_xform3(ib);

  float w = pow2f(emax - 30);
#pragma unroll
  for (int i = 0; i < 64; i++) f[i] = w * (float)ib[i];
}

// ---------------------------------------------------------------- partial blocks
// Padding rule for a 4-vector of which the first n entries are valid
// (encode.cuh:17-38): n=1 -> (a,a,a,a), n=2 -> (a,b,b,a), n=3 -> (a,b,c,a).
CSWAP_HD void pad4(float& a, float& b, float& c, float& d, unsigned n)
{
  if (n == 0) a = 0.0f;
  if (n <= 1) b = a;
  if (n <= 2) c = b;
  if (n <= 3) d = a;
}

CSWAP_HD void pad_block3(float (&f)[64], unsigned bx, unsigned by, unsigned bz)
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
