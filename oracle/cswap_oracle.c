/*
 * cswap_oracle.c -- TEST INFRASTRUCTURE ONLY.
 *
 * A plain-C, single-threaded restatement of the two algorithms on the
 * compression-before-swap path of CSWAP+ (ISCS-ZJU/CSWAP):
 *
 *   (1) the cuZFP fixed-rate codec for 3-D fp32 fields
 *       (CSWAP+/zfp/encode.cuh, encode3.cuh, decode.cuh, decode3.cuh,
 *        shared.h, constants.h, type_info.cuh), which is bit-compatible with
 *       the zfp 0.5.5 serial codec (CSWAP+/zfp/version.h:9-15);
 *   (2) the zero-value compaction (ZVC) format
 *       (CSWAP+/zfp/compression.cu:9-19,134-318).
 *
 * It exists to check the HIP kernels and to be timed as the CPU baseline.
 * Nothing in the shipped library links, loads or calls it; only tests/,
 * __graft_entry__.smoke() and bench.py's cpu_baseline leg may use it.
 *
 * Parity pins (all in tests/test_oracle_*.py):
 *   orc_zfp_encode3_f32 / orc_zfp_decode3_f32 : byte-exact against streams and
 *       decoded fields produced by the zfp 0.5.5 command-line codec
 *       (tests/golden/, made by tests/golden/make_zfp_golden.py), incl. partial
 *       blocks, all-zero blocks and rates 4/8/16, plus SHA-256 digests of the
 *       16 MiB configuration.
 *   orc_fwd_lift / orc_inv_lift : exact integer matrices on multiples of 16/4,
 *       near-inverse bound, wrap-around brute force.
 *   orc_int2uint / orc_uint2int : bijection + negabinary closed form.
 *   orc_perm3 : permutation sorted by (i+j+k, i^2+j^2+k^2).
 *   orc_zfp_encode2/decode2/encode1/decode1 : byte-exact against zfp 0.5.5 2-D and
 *       1-D golden vectors (tests/golden/zfp_golden_12d.npz).
 *   orc_zfp_encode_i32 / orc_zfp_decode_i32 : byte-exact against zfp 0.5.5 -t i32
 *       vectors of 1, 2 and 3 dimensions (tests/golden/zfp_golden_i32.npz).
 *   orc_zfp_encode_64 / orc_zfp_decode_64 : byte-exact against zfp 0.5.5 -d and
 *       -t i64 vectors of 1, 2 and 3 dimensions (tests/golden/zfp_golden_64.npz).
 *   all of the ZFP entry points above, additionally: byte-exact against the stock
 *       zfp 0.5.5 library itself (where the machine has it) on fields of a few
 *       hundred thousand values of every scalar type and dimensionality.
 *   orc_zvc_* : numpy boolean indexing / packbits / cumsum.
 *
 * Undefined in the reference and therefore unpinned here: blocks whose largest
 * magnitude is non-zero but below 2^-97 (the float scale factor 2^(30-emax)
 * overflows, CSWAP+/zfp/encode.cuh:127-132; for doubles below 2^-961, where in
 * addition the cast to int64 is made saturating here), NaN/Inf inputs to the ZFP path,
 * and ZVC mask words past the end of a partially filled last chunk.
 */
#include <math.h>
#include <stdint.h>
#include <stddef.h>
#include <string.h>
#include <stdlib.h>
#ifdef _OPENMP
#include <omp.h>
#endif

typedef uint64_t word_t;

/* threads the multi-threaded build will use (1 for the serial build) */
int orc_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* ------------------------------------------------------------------------ */
/* bit stream: 64-bit little-endian words, bit j of the stream is bit j%64   */
/* of word j/64 (CSWAP+/zfp/shared.h:5, bitstream.c:237-311).                 */
/* ------------------------------------------------------------------------ */

typedef struct {
    word_t *words;
    size_t pos; /* absolute bit position of the next bit */
} bitcur;

/* append the low n (0..64) bits of v, LSB first.  The reference adds into a
 * zeroed stream with atomicAdd (encode.cuh:252-283); on zeroed, non-overlapping
 * bit ranges that is a bitwise OR. */
static void put_bits(bitcur *c, word_t v, unsigned n)
{
    if (n == 0) return;
    if (n < 64) v &= (((word_t)1) << n) - 1;
    size_t w = c->pos >> 6;
    unsigned s = (unsigned)(c->pos & 63);
    c->words[w] |= v << s;
    if (s + n > 64) c->words[w + 1] |= v >> (64 - s);
    c->pos += n;
}

static unsigned get_bit(bitcur *c)
{
    unsigned b = (unsigned)((c->words[c->pos >> 6] >> (c->pos & 63)) & 1u);
    c->pos++;
    return b;
}

/* read n (0..64) bits, LSB first (decode.cuh:92-123). */
static word_t get_bits(bitcur *c, unsigned n)
{
    if (n == 0) return 0;
    size_t w = c->pos >> 6;
    unsigned s = (unsigned)(c->pos & 63);
    word_t v = c->words[w] >> s;
    if (s + n > 64) v |= c->words[w + 1] << (64 - s);
    if (n < 64) v &= (((word_t)1) << n) - 1;
    c->pos += n;
    return v;
}

/* ------------------------------------------------------------------------ */
/* block primitives                                                          */
/* ------------------------------------------------------------------------ */

/* sequency ordering of the 64 coefficients of a 4x4x4 block
 * (constants.h:8-93): ascending i+j+k, ties by i^2+j^2+k^2, remaining ties in
 * the order the reference table lists them.  The table is data, written here
 * as (x,y,z) triples packed as x + 4y + 16z. */
#define P3(x, y, z) ((unsigned char)((x) + 4 * ((y) + 4 * (z))))
static const unsigned char PERM3[64] = {
    P3(0,0,0),
    P3(1,0,0), P3(0,1,0), P3(0,0,1),
    P3(0,1,1), P3(1,0,1), P3(1,1,0),
    P3(2,0,0), P3(0,2,0), P3(0,0,2),
    P3(1,1,1),
    P3(2,1,0), P3(2,0,1), P3(0,2,1), P3(1,2,0), P3(1,0,2), P3(0,1,2),
    P3(3,0,0), P3(0,3,0), P3(0,0,3),
    P3(2,1,1), P3(1,2,1), P3(1,1,2),
    P3(0,2,2), P3(2,0,2), P3(2,2,0),
    P3(3,1,0), P3(3,0,1), P3(0,3,1), P3(1,3,0), P3(1,0,3), P3(0,1,3),
    P3(1,2,2), P3(2,1,2), P3(2,2,1),
    P3(3,1,1), P3(1,3,1), P3(1,1,3),
    P3(3,2,0), P3(3,0,2), P3(0,3,2), P3(2,3,0), P3(2,0,3), P3(0,2,3),
    P3(2,2,2),
    P3(3,2,1), P3(3,1,2), P3(1,3,2), P3(2,3,1), P3(2,1,3), P3(1,2,3),
    P3(0,3,3), P3(3,0,3), P3(3,3,0),
    P3(3,2,2), P3(2,3,2), P3(2,2,3),
    P3(1,3,3), P3(3,1,3), P3(3,3,1),
    P3(2,3,3), P3(3,2,3), P3(3,3,2),
    P3(3,3,3),
};
#undef P3

void orc_perm3(unsigned char out[64]) { memcpy(out, PERM3, 64); }

/* two's complement <-> negabinary (shared.h:168-181, decode.cuh:26-37) */
uint32_t orc_int2uint(int32_t x)
{
    return ((uint32_t)x + 0xaaaaaaaau) ^ 0xaaaaaaaau;
}
int32_t orc_uint2int(uint32_t u)
{
    return (int32_t)((u ^ 0xaaaaaaaau) - 0xaaaaaaaau);
}

/* int32 arithmetic that wraps like the GPU's (no signed-overflow UB). */
static inline int32_t wadd(int32_t a, int32_t b) { return (int32_t)((uint32_t)a + (uint32_t)b); }
static inline int32_t wsub(int32_t a, int32_t b) { return (int32_t)((uint32_t)a - (uint32_t)b); }
static inline int32_t wshl1(int32_t a) { return (int32_t)((uint32_t)a << 1); }
static inline int32_t asr1(int32_t a) { return a >> 1; } /* arithmetic on gcc/clang */

/* forward lifting of one 4-vector with element stride s (encode.cuh:73-99) */
void orc_fwd_lift(int32_t *p, ptrdiff_t s)
{
    int32_t x = p[0], y = p[s], z = p[2 * s], w = p[3 * s];
    x = wadd(x, w); x = asr1(x); w = wsub(w, x);
    z = wadd(z, y); z = asr1(z); y = wsub(y, z);
    x = wadd(x, z); x = asr1(x); z = wsub(z, x);
    w = wadd(w, y); w = asr1(w); y = wsub(y, w);
    w = wadd(w, asr1(y)); y = wsub(y, asr1(w));
    p[0] = x; p[s] = y; p[2 * s] = z; p[3 * s] = w;
}

/* inverse lifting (shared.h:217-248) */
void orc_inv_lift(int32_t *p, ptrdiff_t s)
{
    int32_t x = p[0], y = p[s], z = p[2 * s], w = p[3 * s];
    y = wadd(y, asr1(w)); w = wsub(w, asr1(y));
    y = wadd(y, w); w = wshl1(w); w = wsub(w, y);
    z = wadd(z, x); x = wshl1(x); x = wsub(x, z);
    y = wadd(y, z); z = wshl1(z); z = wsub(z, y);
    w = wadd(w, x); x = wshl1(x); x = wsub(x, w);
    p[0] = x; p[s] = y; p[2 * s] = z; p[3 * s] = w;
}

/* 3-D transform order: x, then y, then z (encode.cuh:154-175); inverse is
 * z, y, x (decode.cuh:184-201). */
void orc_fwd_xform3(int32_t *b)
{
    int x, y, z;
    for (z = 0; z < 4; z++) for (y = 0; y < 4; y++) orc_fwd_lift(b + 4 * y + 16 * z, 1);
    for (x = 0; x < 4; x++) for (z = 0; z < 4; z++) orc_fwd_lift(b + 16 * z + x, 4);
    for (y = 0; y < 4; y++) for (x = 0; x < 4; x++) orc_fwd_lift(b + x + 4 * y, 16);
}
void orc_inv_xform3(int32_t *b)
{
    int x, y, z;
    for (y = 0; y < 4; y++) for (x = 0; x < 4; x++) orc_inv_lift(b + x + 4 * y, 16);
    for (x = 0; x < 4; x++) for (z = 0; z < 4; z++) orc_inv_lift(b + 16 * z + x, 4);
    for (z = 0; z < 4; z++) for (y = 0; y < 4; y++) orc_inv_lift(b + 4 * y + 16 * z, 1);
}

/* block exponent (encode.cuh:40-71): frexp exponent of the largest magnitude,
 * -127 for an all-zero block, clamped to >= -126 for subnormals. */
static int block_emax_n(const float *f, int count);
int orc_block_emax(const float *f) { return block_emax_n(f, 64); }
static int block_emax_n(const float *f, int count)
{
    float m = 0.0f;
    for (int i = 0; i < count; i++) m = fmaxf(m, fabsf(f[i]));
    int e = -127;
    if (m > 0.0f) {
        frexpf(m, &e);
        if (e < -126) e = -126;
    }
    return e;
}

/* block-floating-point cast (encode.cuh:120-149): scale by 2^(30-emax) held
 * as a float, multiply in float, truncate toward zero. */
void orc_fwd_cast(int32_t *ib, const float *fb, int emax)
{
    float s = (float)ldexp(1.0, 30 - emax);
    for (int i = 0; i < 64; i++) ib[i] = (int32_t)(s * fb[i]);
}

/* embedded bit-plane coder (encode.cuh:306-345).  budget = bits available for
 * the 64 coefficients; returns the number of bits written. */
static unsigned encode_ints(bitcur *c, unsigned budget, const uint32_t *u, unsigned size)
{
    unsigned bits = budget;
    unsigned n = 0;
    for (int k = 31; k >= 0 && bits; k--) {
        /* gather bit plane k: bit i of x is bit k of u[i] */
        word_t x = 0;
        for (unsigned i = 0; i < size; i++) x |= (word_t)((u[i] >> k) & 1u) << i;
        /* first n coefficients are already significant: verbatim */
        unsigned m = n < bits ? n : bits;
        bits -= m;
        put_bits(c, x, m);
        x = (m < 64) ? (x >> m) : 0;
        /* group tests + unary run lengths for the rest */
        while (n < size && bits) {
            bits--;
            unsigned any = (x != 0);
            put_bits(c, any, 1);
            if (!any) break;
            while (n < size - 1 && bits) {
                bits--;
                unsigned b = (unsigned)(x & 1u);
                put_bits(c, b, 1);
                if (b) break;
                x >>= 1; n++;
            }
            x >>= 1; n++;
        }
    }
    return budget - bits;
}

/* mirror of the coder (decode.cuh:127-179) */
static void decode_ints(bitcur *c, unsigned budget, uint32_t *u, unsigned size)
{
    unsigned bits = budget;
    unsigned n = 0;
    memset(u, 0, size * sizeof(uint32_t));
    for (int k = 31; k >= 0 && bits; k--) {
        unsigned m = n < bits ? n : bits;
        bits -= m;
        word_t x = get_bits(c, m);
        while (bits && n < size) {
            bits--;
            if (!get_bit(c)) break;
            while (bits && n < size - 1) {
                bits--;
                if (get_bit(c)) break;
                n++;
            }
            x += (word_t)1 << n;
            n++;
        }
        for (unsigned i = 0; i < size; i++, x >>= 1) u[i] += (uint32_t)(x & 1u) << k;
    }
}

/* one block: header + payload at bit offset block_idx*maxbits
 * (encode.cuh:347-368).  fb holds the gathered (and padded) 64 values. */
void orc_zfp_encode_block_f32(const float *fb, unsigned maxbits, size_t block_idx, word_t *stream)
{
    bitcur c = { stream, block_idx * (size_t)maxbits };
    int emax = orc_block_emax(fb);
    unsigned e = (unsigned)(emax + 127); /* maxprec is 32 for every float exponent */
    if (!e) return;                      /* all-zero block: leave zero bits */
    put_bits(&c, 2 * e + 1, 9);
    int32_t ib[64];
    uint32_t ub[64];
    orc_fwd_cast(ib, fb, emax);
    orc_fwd_xform3(ib);
    for (int i = 0; i < 64; i++) ub[i] = orc_int2uint(ib[PERM3[i]]);
    encode_ints(&c, maxbits - 9, ub, 64);
}

/* decode.cuh:228-288; fb is left untouched (caller pre-zeroes) for an empty block */
void orc_zfp_decode_block_f32(const word_t *stream, unsigned maxbits, size_t block_idx, float *fb)
{
    bitcur c = { (word_t *)stream, block_idx * (size_t)maxbits };
    if (!get_bit(&c)) return;
    int emax = (int)get_bits(&c, 8) - 127;
    uint32_t ub[64];
    int32_t ib[64];
    decode_ints(&c, maxbits - 9, ub, 64);
    for (int i = 0; i < 64; i++) ib[PERM3[i]] = orc_uint2int(ub[i]);
    orc_inv_xform3(ib);
    float w = ldexpf(1.0f, emax - 30);
    for (int i = 0; i < 64; i++) fb[i] = w * (float)ib[i];
}

/* ------------------------------------------------------------------------ */
/* field level                                                               */
/* ------------------------------------------------------------------------ */

static size_t pad4(size_t n) { return (n + 3) & ~(size_t)3; }

/* encode3.cuh:128-133 and shared.h:73-84: whole 64-bit words, rounded DOWN */
size_t orc_zfp_stream_bytes3(size_t nx, size_t ny, size_t nz, unsigned maxbits)
{
    size_t blocks = pad4(nx) * pad4(ny) * pad4(nz) / 64;
    return (blocks * (size_t)maxbits / 64) * sizeof(word_t);
}

/* partial-block padding rule (encode.cuh:17-38) applied to a 4-vector of
 * which the first n entries are valid */
static void pad_vec(float *p, unsigned n, ptrdiff_t s)
{
    switch (n) {
    case 0: p[0] = 0; /* fall through */
    case 1: p[s] = p[0]; /* fall through */
    case 2: p[2 * s] = p[s]; /* fall through */
    case 3: p[3 * s] = p[0]; /* fall through */
    default: break;
    }
}

/* gather one block at (x0,y0,z0) with extents (bx,by,bz) in 1..4
 * (encode3.cuh:12-47) */
static void gather3(float *q, const float *p, unsigned bx, unsigned by, unsigned bz,
                    ptrdiff_t sx, ptrdiff_t sy, ptrdiff_t sz)
{
    unsigned x, y, z;
    for (z = 0; z < bz; z++) {
        for (y = 0; y < by; y++) {
            for (x = 0; x < bx; x++) q[16 * z + 4 * y + x] = p[x * sx + y * sy + z * sz];
            pad_vec(q + 16 * z + 4 * y, bx, 1);
        }
        for (x = 0; x < 4; x++) pad_vec(q + 16 * z + x, by, 4);
    }
    for (y = 0; y < 4; y++)
        for (x = 0; x < 4; x++) pad_vec(q + 4 * y + x, bz, 16);
}

/* Compress a 3-D field a[nz][ny][nx] with element strides (0 = contiguous
 * default, cuZFP.cu:372-375).  Blocks are numbered x fastest
 * (encode3.cuh:79-87).  Returns the stream size in bytes; the stream must hold
 * ceil(blocks*maxbits/64) words and is zeroed here (encode3.cuh:152). */
size_t orc_zfp_encode3_f32(const float *in, size_t nx, size_t ny, size_t nz,
                           ptrdiff_t sx, ptrdiff_t sy, ptrdiff_t sz,
                           unsigned maxbits, word_t *stream)
{
    if (!sx) sx = 1;
    if (!sy) sy = (ptrdiff_t)nx;
    if (!sz) sz = (ptrdiff_t)(nx * ny);
    size_t mx = pad4(nx) / 4, my = pad4(ny) / 4, mz = pad4(nz) / 4;
    size_t blocks = mx * my * mz;
    size_t words = (blocks * (size_t)maxbits + 63) / 64;
    memset(stream, 0, words * sizeof(word_t));
    /* blocks are independent; with whole-word blocks they also touch disjoint
     * words, so the multi-threaded build (liboracle_omp.so, used only for the
     * all-cores CPU baseline) may split this loop */
#ifdef _OPENMP
#pragma omp parallel for schedule(static) if (maxbits % 64 == 0)
#endif
    for (size_t b = 0; b < blocks; b++) {
        float fb[64];
        size_t x0 = (b % mx) * 4, y0 = ((b / mx) % my) * 4, z0 = (b / (mx * my)) * 4;
        unsigned bx = (unsigned)(nx - x0 < 4 ? nx - x0 : 4);
        unsigned by = (unsigned)(ny - y0 < 4 ? ny - y0 : 4);
        unsigned bz = (unsigned)(nz - z0 < 4 ? nz - z0 : 4);
        gather3(fb, in + (ptrdiff_t)x0 * sx + (ptrdiff_t)y0 * sy + (ptrdiff_t)z0 * sz,
                bx, by, bz, sx, sy, sz);
        orc_zfp_encode_block_f32(fb, maxbits, b, stream);
    }
    return orc_zfp_stream_bytes3(nx, ny, nz, maxbits);
}

/* decode3.cuh:42-107: empty blocks decode to +0.0, partial blocks store only
 * their valid part. */
void orc_zfp_decode3_f32(const word_t *stream, size_t nx, size_t ny, size_t nz,
                         ptrdiff_t sx, ptrdiff_t sy, ptrdiff_t sz,
                         unsigned maxbits, float *out)
{
    if (!sx) sx = 1;
    if (!sy) sy = (ptrdiff_t)nx;
    if (!sz) sz = (ptrdiff_t)(nx * ny);
    size_t mx = pad4(nx) / 4, my = pad4(ny) / 4, mz = pad4(nz) / 4;
    size_t blocks = mx * my * mz;
#ifdef _OPENMP
#pragma omp parallel for schedule(static)
#endif
    for (size_t b = 0; b < blocks; b++) {
        float fb[64];
        size_t x0 = (b % mx) * 4, y0 = ((b / mx) % my) * 4, z0 = (b / (mx * my)) * 4;
        unsigned bx = (unsigned)(nx - x0 < 4 ? nx - x0 : 4);
        unsigned by = (unsigned)(ny - y0 < 4 ? ny - y0 : 4);
        unsigned bz = (unsigned)(nz - z0 < 4 ? nz - z0 : 4);
        memset(fb, 0, sizeof fb);
        orc_zfp_decode_block_f32(stream, maxbits, b, fb);
        float *p = out + (ptrdiff_t)x0 * sx + (ptrdiff_t)y0 * sy + (ptrdiff_t)z0 * sz;
        for (unsigned z = 0; z < bz; z++)
            for (unsigned y = 0; y < by; y++)
                for (unsigned x = 0; x < bx; x++)
                    p[x * sx + y * sy + z * sz] = fb[16 * z + 4 * y + x];
    }
}

/* ------------------------------------------------------------------------ */
/* 2-D and 1-D fields (encode2.cuh, encode1.cuh, decode2.cuh, decode1.cuh):    */
/* blocks of 4x4 = 16 and 4 values, coefficient order perm_2 / identity       */
/* (constants.h:95-133), transform along x then y (encode.cuh:177-201).        */
/* ------------------------------------------------------------------------ */

#define P2(i, j) ((unsigned char)((i) + 4 * (j)))
static const unsigned char PERM2[16] = {
    P2(0,0), P2(1,0), P2(0,1), P2(1,1), P2(2,0), P2(0,2), P2(2,1), P2(1,2),
    P2(3,0), P2(0,3), P2(2,2), P2(3,1), P2(1,3), P2(3,2), P2(2,3), P2(3,3),
};
#undef P2
void orc_perm2(unsigned char out[16]) { memcpy(out, PERM2, 16); }

/* dims = 1 or 2; fb holds 4 or 16 gathered (and padded) values */
static void encode_block_low(const float *fb, int dims, unsigned maxbits, size_t block_idx, word_t *stream)
{
    const int size = dims == 2 ? 16 : 4;
    bitcur c = { stream, block_idx * (size_t)maxbits };
    int emax = block_emax_n(fb, size);
    unsigned e = (unsigned)(emax + 127);
    if (!e) return;
    put_bits(&c, 2 * e + 1, 9);
    int32_t ib[16];
    uint32_t ub[16];
    float s = (float)ldexp(1.0, 30 - emax);
    for (int i = 0; i < size; i++) ib[i] = (int32_t)(s * fb[i]);
    if (dims == 2) {
        for (int y = 0; y < 4; y++) orc_fwd_lift(ib + 4 * y, 1);
        for (int x = 0; x < 4; x++) orc_fwd_lift(ib + x, 4);
        for (int i = 0; i < 16; i++) ub[i] = orc_int2uint(ib[PERM2[i]]);
    } else {
        orc_fwd_lift(ib, 1);
        for (int i = 0; i < 4; i++) ub[i] = orc_int2uint(ib[i]);
    }
    encode_ints(&c, maxbits - 9, ub, (unsigned)size);
}

static void decode_block_low(const word_t *stream, int dims, unsigned maxbits, size_t block_idx, float *fb)
{
    const int size = dims == 2 ? 16 : 4;
    bitcur c = { (word_t *)stream, block_idx * (size_t)maxbits };
    if (!get_bit(&c)) return;
    int emax = (int)get_bits(&c, 8) - 127;
    uint32_t ub[16];
    int32_t ib[16];
    decode_ints(&c, maxbits - 9, ub, (unsigned)size);
    if (dims == 2) {
        for (int i = 0; i < 16; i++) ib[PERM2[i]] = orc_uint2int(ub[i]);
        for (int x = 0; x < 4; x++) orc_inv_lift(ib + x, 4);     /* decode.cuh:203-214: y first, then x */
        for (int y = 0; y < 4; y++) orc_inv_lift(ib + 4 * y, 1);
    } else {
        for (int i = 0; i < 4; i++) ib[i] = orc_uint2int(ub[i]);
        orc_inv_lift(ib, 1);
    }
    float w = ldexpf(1.0f, emax - 30);
    for (int i = 0; i < size; i++) fb[i] = w * (float)ib[i];
}

/* stream sizes: whole words, rounded UP for 1-D and 2-D (shared.h:42-71) */
size_t orc_zfp_stream_bytes2(size_t nx, size_t ny, unsigned maxbits)
{
    size_t blocks = pad4(nx) * pad4(ny) / 16;
    return ((blocks * (size_t)maxbits + 63) / 64) * sizeof(word_t);
}
size_t orc_zfp_stream_bytes1(size_t nx, unsigned maxbits)
{
    size_t blocks = pad4(nx) / 4;
    return ((blocks * (size_t)maxbits + 63) / 64) * sizeof(word_t);
}

size_t orc_zfp_encode2_f32(const float *in, size_t nx, size_t ny, ptrdiff_t sx, ptrdiff_t sy,
                           unsigned maxbits, word_t *stream)
{
    if (!sx) sx = 1;
    if (!sy) sy = (ptrdiff_t)nx;
    size_t mx = pad4(nx) / 4, my = pad4(ny) / 4, blocks = mx * my;
    memset(stream, 0, ((blocks * (size_t)maxbits + 63) / 64) * sizeof(word_t));
    for (size_t b = 0; b < blocks; b++) {
        float fb[16];
        size_t x0 = (b % mx) * 4, y0 = (b / mx) * 4;
        unsigned bx = (unsigned)(nx - x0 < 4 ? nx - x0 : 4), by = (unsigned)(ny - y0 < 4 ? ny - y0 : 4);
        const float *p = in + (ptrdiff_t)x0 * sx + (ptrdiff_t)y0 * sy;
        for (unsigned y = 0; y < by; y++) {
            for (unsigned x = 0; x < bx; x++) fb[4 * y + x] = p[x * sx + y * sy];
            pad_vec(fb + 4 * y, bx, 1);
        }
        for (unsigned x = 0; x < 4; x++) pad_vec(fb + x, by, 4);
        encode_block_low(fb, 2, maxbits, b, stream);
    }
    return orc_zfp_stream_bytes2(nx, ny, maxbits);
}

void orc_zfp_decode2_f32(const word_t *stream, size_t nx, size_t ny, ptrdiff_t sx, ptrdiff_t sy,
                         unsigned maxbits, float *out)
{
    if (!sx) sx = 1;
    if (!sy) sy = (ptrdiff_t)nx;
    size_t mx = pad4(nx) / 4, my = pad4(ny) / 4, blocks = mx * my;
    for (size_t b = 0; b < blocks; b++) {
        float fb[16];
        size_t x0 = (b % mx) * 4, y0 = (b / mx) * 4;
        unsigned bx = (unsigned)(nx - x0 < 4 ? nx - x0 : 4), by = (unsigned)(ny - y0 < 4 ? ny - y0 : 4);
        memset(fb, 0, sizeof fb);
        decode_block_low(stream, 2, maxbits, b, fb);
        float *p = out + (ptrdiff_t)x0 * sx + (ptrdiff_t)y0 * sy;
        for (unsigned y = 0; y < by; y++)
            for (unsigned x = 0; x < bx; x++) p[x * sx + y * sy] = fb[4 * y + x];
    }
}

size_t orc_zfp_encode1_f32(const float *in, size_t nx, ptrdiff_t sx, unsigned maxbits, word_t *stream)
{
    if (!sx) sx = 1;
    size_t blocks = pad4(nx) / 4;
    memset(stream, 0, ((blocks * (size_t)maxbits + 63) / 64) * sizeof(word_t));
    for (size_t b = 0; b < blocks; b++) {
        float fb[4];
        size_t x0 = b * 4;
        unsigned bx = (unsigned)(nx - x0 < 4 ? nx - x0 : 4);
        for (unsigned x = 0; x < bx; x++) fb[x] = in[(ptrdiff_t)(x0 + x) * sx];
        pad_vec(fb, bx, 1);
        encode_block_low(fb, 1, maxbits, b, stream);
    }
    return orc_zfp_stream_bytes1(nx, maxbits);
}

void orc_zfp_decode1_f32(const word_t *stream, size_t nx, ptrdiff_t sx, unsigned maxbits, float *out)
{
    if (!sx) sx = 1;
    size_t blocks = pad4(nx) / 4;
    for (size_t b = 0; b < blocks; b++) {
        float fb[4] = {0, 0, 0, 0};
        size_t x0 = b * 4;
        unsigned bx = (unsigned)(nx - x0 < 4 ? nx - x0 : 4);
        decode_block_low(stream, 1, maxbits, b, fb);
        for (unsigned x = 0; x < bx; x++) out[(ptrdiff_t)(x0 + x) * sx] = fb[x];
    }
}

/* ------------------------------------------------------------------------ */
/* int32 fields (zfp_type_int32, cuZFP.cu:412-416,513-517): the same transform */
/* and coder applied to the values themselves -- no exponent header, no cast,  */
/* the whole maxbits is the coder's budget (encode.cuh:371-380,393-402,415-424;*/
/* decode.cuh:228-288 with the integer specialisations).  Partial blocks are   */
/* padded by the same rule.  dims = 1, 2 or 3.                                 */
/* ------------------------------------------------------------------------ */

static void pad_vec_i32(int32_t *p, unsigned n, ptrdiff_t s)
{
    switch (n) {
    case 0: p[0] = 0; /* fall through */
    case 1: p[s] = p[0]; /* fall through */
    case 2: p[2 * s] = p[s]; /* fall through */
    case 3: p[3 * s] = p[0]; /* fall through */
    default: break;
    }
}

static void encode_block_i32(int32_t *ib, int dims, unsigned maxbits, size_t block_idx, word_t *stream)
{
    bitcur c = { stream, block_idx * (size_t)maxbits };
    uint32_t ub[64];
    if (dims == 3) {
        orc_fwd_xform3(ib);
        for (int i = 0; i < 64; i++) ub[i] = orc_int2uint(ib[PERM3[i]]);
        encode_ints(&c, maxbits, ub, 64);
    } else if (dims == 2) {
        for (int y = 0; y < 4; y++) orc_fwd_lift(ib + 4 * y, 1);
        for (int x = 0; x < 4; x++) orc_fwd_lift(ib + x, 4);
        for (int i = 0; i < 16; i++) ub[i] = orc_int2uint(ib[PERM2[i]]);
        encode_ints(&c, maxbits, ub, 16);
    } else {
        orc_fwd_lift(ib, 1);
        for (int i = 0; i < 4; i++) ub[i] = orc_int2uint(ib[i]);
        encode_ints(&c, maxbits, ub, 4);
    }
}

static void decode_block_i32(const word_t *stream, int dims, unsigned maxbits, size_t block_idx, int32_t *ib)
{
    bitcur c = { (word_t *)stream, block_idx * (size_t)maxbits };
    uint32_t ub[64];
    if (dims == 3) {
        decode_ints(&c, maxbits, ub, 64);
        for (int i = 0; i < 64; i++) ib[PERM3[i]] = orc_uint2int(ub[i]);
        orc_inv_xform3(ib);
    } else if (dims == 2) {
        decode_ints(&c, maxbits, ub, 16);
        for (int i = 0; i < 16; i++) ib[PERM2[i]] = orc_uint2int(ub[i]);
        for (int x = 0; x < 4; x++) orc_inv_lift(ib + x, 4);
        for (int y = 0; y < 4; y++) orc_inv_lift(ib + 4 * y, 1);
    } else {
        decode_ints(&c, maxbits, ub, 4);
        for (int i = 0; i < 4; i++) ib[i] = orc_uint2int(ub[i]);
        orc_inv_lift(ib, 1);
    }
}

/* a[nz][ny][nx] (ny, nz ignored below dims); strides 0 = contiguous.  Returns
 * the stream size in bytes as the reference reports it. */
size_t orc_zfp_encode_i32(const int32_t *in, int dims, size_t nx, size_t ny, size_t nz,
                          ptrdiff_t sx, ptrdiff_t sy, ptrdiff_t sz, unsigned maxbits, word_t *stream)
{
    if (dims < 2) ny = 1;
    if (dims < 3) nz = 1;
    if (!sx) sx = 1;
    if (!sy) sy = (ptrdiff_t)nx;
    if (!sz) sz = (ptrdiff_t)(nx * ny);
    size_t mx = pad4(nx) / 4, my = dims >= 2 ? pad4(ny) / 4 : 1, mz = dims >= 3 ? pad4(nz) / 4 : 1;
    size_t blocks = mx * my * mz;
    memset(stream, 0, ((blocks * (size_t)maxbits + 63) / 64) * sizeof(word_t));
    for (size_t b = 0; b < blocks; b++) {
        int32_t q[64];
        size_t x0 = (b % mx) * 4, y0 = ((b / mx) % my) * 4, z0 = (b / (mx * my)) * 4;
        unsigned bx = (unsigned)(nx - x0 < 4 ? nx - x0 : 4);
        unsigned by = dims >= 2 ? (unsigned)(ny - y0 < 4 ? ny - y0 : 4) : 1;
        unsigned bz = dims >= 3 ? (unsigned)(nz - z0 < 4 ? nz - z0 : 4) : 1;
        const int32_t *p = in + (ptrdiff_t)x0 * sx + (ptrdiff_t)y0 * sy + (ptrdiff_t)z0 * sz;
        memset(q, 0, sizeof q);
        for (unsigned z = 0; z < bz; z++) {
            for (unsigned y = 0; y < by; y++) {
                for (unsigned x = 0; x < bx; x++) q[16 * z + 4 * y + x] = p[x * sx + y * sy + z * sz];
                pad_vec_i32(q + 16 * z + 4 * y, bx, 1);
            }
            if (dims >= 2)
                for (unsigned x = 0; x < 4; x++) pad_vec_i32(q + 16 * z + x, by, 4);
        }
        if (dims >= 3)
            for (unsigned y = 0; y < 4; y++)
                for (unsigned x = 0; x < 4; x++) pad_vec_i32(q + 4 * y + x, bz, 16);
        encode_block_i32(q, dims, maxbits, b, stream);
    }
    if (dims == 3) return orc_zfp_stream_bytes3(nx, ny, nz, maxbits);
    return ((blocks * (size_t)maxbits + 63) / 64) * sizeof(word_t);
}

void orc_zfp_decode_i32(const word_t *stream, int dims, size_t nx, size_t ny, size_t nz,
                        ptrdiff_t sx, ptrdiff_t sy, ptrdiff_t sz, unsigned maxbits, int32_t *out)
{
    if (dims < 2) ny = 1;
    if (dims < 3) nz = 1;
    if (!sx) sx = 1;
    if (!sy) sy = (ptrdiff_t)nx;
    if (!sz) sz = (ptrdiff_t)(nx * ny);
    size_t mx = pad4(nx) / 4, my = dims >= 2 ? pad4(ny) / 4 : 1, mz = dims >= 3 ? pad4(nz) / 4 : 1;
    size_t blocks = mx * my * mz;
    for (size_t b = 0; b < blocks; b++) {
        int32_t q[64];
        size_t x0 = (b % mx) * 4, y0 = ((b / mx) % my) * 4, z0 = (b / (mx * my)) * 4;
        unsigned bx = (unsigned)(nx - x0 < 4 ? nx - x0 : 4);
        unsigned by = dims >= 2 ? (unsigned)(ny - y0 < 4 ? ny - y0 : 4) : 1;
        unsigned bz = dims >= 3 ? (unsigned)(nz - z0 < 4 ? nz - z0 : 4) : 1;
        memset(q, 0, sizeof q);
        decode_block_i32(stream, dims, maxbits, b, q);
        int32_t *p = out + (ptrdiff_t)x0 * sx + (ptrdiff_t)y0 * sy + (ptrdiff_t)z0 * sz;
        for (unsigned z = 0; z < bz; z++)
            for (unsigned y = 0; y < by; y++)
                for (unsigned x = 0; x < bx; x++) p[x * sx + y * sy + z * sz] = q[16 * z + 4 * y + x];
    }
}

/* ------------------------------------------------------------------------ */
/* 64-bit element types (zfp_type_double, zfp_type_int64; cuZFP.cu:401-423,   */
/* 479-504).  Same structure with 64-bit integers and 64 bit planes:          */
/*   double: 12 header bits (flag + 11-bit biased exponent, type_info.cuh:8-17),*/
/*           scale 2^(62-emax) (encode.cuh:136-149), block precision           */
/*           min(64, emax + 1074 + 8) (encode.cuh:10-15 -- the "+ 8" is used   */
/*           for every dimensionality), so blocks whose largest magnitude is   */
/*           below 2^-1018 code fewer than 64 planes; the decoder always reads */
/*           down to plane 0 (decode.cuh:131-133), which finds zero bits there.*/
/*   int64 : no header, no cast (encode.cuh:382-391 and the 1-D/2-D twins).    */
/* Conversions double -> int64 saturate (what the reference's GPU does for the */
/* overflowing scale of near-subnormal blocks; C leaves them undefined).      */
/* Values travel as 64-bit patterns.                                          */
/* ------------------------------------------------------------------------ */

#define NB64 0xaaaaaaaaaaaaaaaaull

static inline int64_t wadd64(int64_t a, int64_t b) { return (int64_t)((uint64_t)a + (uint64_t)b); }
static inline int64_t wsub64(int64_t a, int64_t b) { return (int64_t)((uint64_t)a - (uint64_t)b); }
static inline int64_t wshl64(int64_t a) { return (int64_t)((uint64_t)a << 1); }
static inline int64_t asr64(int64_t a) { return a >> 1; }

static void fwd_lift64(int64_t *p, ptrdiff_t s)
{
    int64_t x = p[0], y = p[s], z = p[2 * s], w = p[3 * s];
    x = wadd64(x, w); x = asr64(x); w = wsub64(w, x);
    z = wadd64(z, y); z = asr64(z); y = wsub64(y, z);
    x = wadd64(x, z); x = asr64(x); z = wsub64(z, x);
    w = wadd64(w, y); w = asr64(w); y = wsub64(y, w);
    w = wadd64(w, asr64(y)); y = wsub64(y, asr64(w));
    p[0] = x; p[s] = y; p[2 * s] = z; p[3 * s] = w;
}

static void inv_lift64(int64_t *p, ptrdiff_t s)
{
    int64_t x = p[0], y = p[s], z = p[2 * s], w = p[3 * s];
    y = wadd64(y, asr64(w)); w = wsub64(w, asr64(y));
    y = wadd64(y, w); w = wshl64(w); w = wsub64(w, y);
    z = wadd64(z, x); x = wshl64(x); x = wsub64(x, z);
    y = wadd64(y, z); z = wshl64(z); z = wsub64(z, y);
    w = wadd64(w, x); x = wshl64(x); x = wsub64(x, w);
    p[0] = x; p[s] = y; p[2 * s] = z; p[3 * s] = w;
}

static void fwd_xform64(int64_t *b, int dims)
{
    int x, y, z;
    if (dims == 3) {
        for (z = 0; z < 4; z++) for (y = 0; y < 4; y++) fwd_lift64(b + 4 * y + 16 * z, 1);
        for (x = 0; x < 4; x++) for (z = 0; z < 4; z++) fwd_lift64(b + 16 * z + x, 4);
        for (y = 0; y < 4; y++) for (x = 0; x < 4; x++) fwd_lift64(b + x + 4 * y, 16);
    } else if (dims == 2) {
        for (y = 0; y < 4; y++) fwd_lift64(b + 4 * y, 1);
        for (x = 0; x < 4; x++) fwd_lift64(b + x, 4);
    } else {
        fwd_lift64(b, 1);
    }
}

static void inv_xform64(int64_t *b, int dims)
{
    int x, y, z;
    if (dims == 3) {
        for (y = 0; y < 4; y++) for (x = 0; x < 4; x++) inv_lift64(b + x + 4 * y, 16);
        for (x = 0; x < 4; x++) for (z = 0; z < 4; z++) inv_lift64(b + 16 * z + x, 4);
        for (z = 0; z < 4; z++) for (y = 0; y < 4; y++) inv_lift64(b + 4 * y + 16 * z, 1);
    } else if (dims == 2) {
        for (x = 0; x < 4; x++) inv_lift64(b + x, 4);
        for (y = 0; y < 4; y++) inv_lift64(b + 4 * y, 1);
    } else {
        inv_lift64(b, 1);
    }
}

/* the coder of encode.cuh:306-345 on 64-bit coefficients; planes below kmin are not coded */
static void encode_ints64(bitcur *c, unsigned budget, const uint64_t *u, unsigned size, unsigned kmin)
{
    unsigned bits = budget;
    unsigned n = 0;
    for (int k = 63; k >= (int)kmin && bits; k--) {
        word_t x = 0;
        for (unsigned i = 0; i < size; i++) x |= (word_t)((u[i] >> k) & 1u) << i;
        unsigned m = n < bits ? n : bits;
        bits -= m;
        put_bits(c, x, m);
        x = (m < 64) ? (x >> m) : 0;
        while (n < size && bits) {
            bits--;
            unsigned any = (x != 0);
            put_bits(c, any, 1);
            if (!any) break;
            while (n < size - 1 && bits) {
                bits--;
                unsigned b = (unsigned)(x & 1u);
                put_bits(c, b, 1);
                if (b) break;
                x >>= 1; n++;
            }
            x >>= 1; n++;
        }
    }
}

static void decode_ints64(bitcur *c, unsigned budget, uint64_t *u, unsigned size)
{
    unsigned bits = budget;
    unsigned n = 0;
    memset(u, 0, size * sizeof(uint64_t));
    for (int k = 63; k >= 0 && bits; k--) {
        unsigned m = n < bits ? n : bits;
        bits -= m;
        word_t x = get_bits(c, m);
        while (bits && n < size) {
            bits--;
            if (!get_bit(c)) break;
            while (bits && n < size - 1) {
                bits--;
                if (get_bit(c)) break;
                n++;
            }
            x += (word_t)1 << n;
            n++;
        }
        for (unsigned i = 0; i < size; i++, x >>= 1) u[i] += (uint64_t)(x & 1u) << k;
    }
}

static int64_t sat_i64(double v)
{
    if (v != v) return 0;
    if (v >= 9223372036854775808.0) return INT64_MAX;
    if (v <= -9223372036854775808.0) return INT64_MIN;
    return (int64_t)v;
}

static const unsigned char *perm_for(int dims)
{
    static const unsigned char ident[4] = { 0, 1, 2, 3 };
    return dims == 3 ? PERM3 : dims == 2 ? PERM2 : ident;
}

/* q: the gathered and padded block as 64-bit patterns (overwritten) */
static void encode_block_64(uint64_t *q, int is_int, int dims, unsigned maxbits, size_t block_idx, word_t *stream)
{
    const unsigned size = dims == 3 ? 64 : dims == 2 ? 16 : 4;
    bitcur c = { stream, block_idx * (size_t)maxbits };
    int64_t ib[64];
    unsigned budget = maxbits, kmin = 0;
    if (is_int) {
        memcpy(ib, q, size * sizeof(int64_t));
    } else {
        double fb[64], m = 0.0;
        memcpy(fb, q, size * sizeof(double));
        for (unsigned i = 0; i < size; i++) m = fmax(m, fabs(fb[i]));
        int emax = -1023;
        if (m > 0.0) {
            frexp(m, &emax);
            if (emax < -1022) emax = -1022;
        }
        int maxprec = emax + 1074 + 8;
        if (maxprec > 64) maxprec = 64;
        if (maxprec < 0) maxprec = 0;
        unsigned e = maxprec ? (unsigned)(emax + 1023) : 0;
        if (!e) return;
        put_bits(&c, 2 * (word_t)e + 1, 12);
        budget = maxbits - 12;
        kmin = 64 - (unsigned)maxprec;
        double s = ldexp(1.0, 62 - emax);
        for (unsigned i = 0; i < size; i++) ib[i] = sat_i64(s * fb[i]);
    }
    fwd_xform64(ib, dims);
    const unsigned char *perm = perm_for(dims);
    uint64_t ub[64];
    for (unsigned i = 0; i < size; i++) ub[i] = ((uint64_t)ib[perm[i]] + NB64) ^ NB64;
    encode_ints64(&c, budget, ub, size, kmin);
}

/* q receives the block as 64-bit patterns; an empty double block leaves it untouched */
static void decode_block_64(const word_t *stream, int is_int, int dims, unsigned maxbits, size_t block_idx, uint64_t *q)
{
    const unsigned size = dims == 3 ? 64 : dims == 2 ? 16 : 4;
    bitcur c = { (word_t *)stream, block_idx * (size_t)maxbits };
    unsigned budget = maxbits;
    int emax = 0;
    if (!is_int) {
        if (!get_bit(&c)) return;
        emax = (int)get_bits(&c, 11) - 1023;
        budget = maxbits - 12;
    }
    uint64_t ub[64];
    int64_t ib[64];
    decode_ints64(&c, budget, ub, size);
    const unsigned char *perm = perm_for(dims);
    for (unsigned i = 0; i < size; i++) ib[perm[i]] = (int64_t)((ub[i] ^ NB64) - NB64);
    inv_xform64(ib, dims);
    if (is_int) {
        memcpy(q, ib, size * sizeof(int64_t));
    } else {
        double w = ldexp(1.0, emax - 62), fb[64];
        for (unsigned i = 0; i < size; i++) fb[i] = w * (double)ib[i];
        memcpy(q, fb, size * sizeof(double));
    }
}

static void pad_vec_64(uint64_t *p, unsigned n, ptrdiff_t s)
{
    switch (n) {
    case 0: p[0] = 0; /* fall through */
    case 1: p[s] = p[0]; /* fall through */
    case 2: p[2 * s] = p[s]; /* fall through */
    case 3: p[3 * s] = p[0]; /* fall through */
    default: break;
    }
}

/* in: a[nz][ny][nx] of doubles (is_int 0) or int64 (is_int 1); strides in elements, 0 = contiguous */
size_t orc_zfp_encode_64(const void *in_, int is_int, int dims, size_t nx, size_t ny, size_t nz,
                         ptrdiff_t sx, ptrdiff_t sy, ptrdiff_t sz, unsigned maxbits, word_t *stream)
{
    const uint64_t *in = (const uint64_t *)in_;
    if (dims < 2) ny = 1;
    if (dims < 3) nz = 1;
    if (!sx) sx = 1;
    if (!sy) sy = (ptrdiff_t)nx;
    if (!sz) sz = (ptrdiff_t)(nx * ny);
    size_t mx = pad4(nx) / 4, my = dims >= 2 ? pad4(ny) / 4 : 1, mz = dims >= 3 ? pad4(nz) / 4 : 1;
    size_t blocks = mx * my * mz;
    memset(stream, 0, ((blocks * (size_t)maxbits + 63) / 64) * sizeof(word_t));
    for (size_t b = 0; b < blocks; b++) {
        uint64_t q[64];
        size_t x0 = (b % mx) * 4, y0 = ((b / mx) % my) * 4, z0 = (b / (mx * my)) * 4;
        unsigned bx = (unsigned)(nx - x0 < 4 ? nx - x0 : 4);
        unsigned by = dims >= 2 ? (unsigned)(ny - y0 < 4 ? ny - y0 : 4) : 1;
        unsigned bz = dims >= 3 ? (unsigned)(nz - z0 < 4 ? nz - z0 : 4) : 1;
        const uint64_t *p = in + (ptrdiff_t)x0 * sx + (ptrdiff_t)y0 * sy + (ptrdiff_t)z0 * sz;
        memset(q, 0, sizeof q);
        for (unsigned z = 0; z < bz; z++) {
            for (unsigned y = 0; y < by; y++) {
                for (unsigned x = 0; x < bx; x++) q[16 * z + 4 * y + x] = p[x * sx + y * sy + z * sz];
                pad_vec_64(q + 16 * z + 4 * y, bx, 1);
            }
            if (dims >= 2)
                for (unsigned x = 0; x < 4; x++) pad_vec_64(q + 16 * z + x, by, 4);
        }
        if (dims >= 3)
            for (unsigned y = 0; y < 4; y++)
                for (unsigned x = 0; x < 4; x++) pad_vec_64(q + 4 * y + x, bz, 16);
        encode_block_64(q, is_int, dims, maxbits, b, stream);
    }
    if (dims == 3) return orc_zfp_stream_bytes3(nx, ny, nz, maxbits);
    return ((blocks * (size_t)maxbits + 63) / 64) * sizeof(word_t);
}

void orc_zfp_decode_64(const word_t *stream, int is_int, int dims, size_t nx, size_t ny, size_t nz,
                       ptrdiff_t sx, ptrdiff_t sy, ptrdiff_t sz, unsigned maxbits, void *out_)
{
    uint64_t *out = (uint64_t *)out_;
    if (dims < 2) ny = 1;
    if (dims < 3) nz = 1;
    if (!sx) sx = 1;
    if (!sy) sy = (ptrdiff_t)nx;
    if (!sz) sz = (ptrdiff_t)(nx * ny);
    size_t mx = pad4(nx) / 4, my = dims >= 2 ? pad4(ny) / 4 : 1, mz = dims >= 3 ? pad4(nz) / 4 : 1;
    size_t blocks = mx * my * mz;
    for (size_t b = 0; b < blocks; b++) {
        uint64_t q[64];
        size_t x0 = (b % mx) * 4, y0 = ((b / mx) % my) * 4, z0 = (b / (mx * my)) * 4;
        unsigned bx = (unsigned)(nx - x0 < 4 ? nx - x0 : 4);
        unsigned by = dims >= 2 ? (unsigned)(ny - y0 < 4 ? ny - y0 : 4) : 1;
        unsigned bz = dims >= 3 ? (unsigned)(nz - z0 < 4 ? nz - z0 : 4) : 1;
        memset(q, 0, sizeof q);
        decode_block_64(stream, is_int, dims, maxbits, b, q);
        uint64_t *p = out + (ptrdiff_t)x0 * sx + (ptrdiff_t)y0 * sy + (ptrdiff_t)z0 * sz;
        for (unsigned z = 0; z < bz; z++)
            for (unsigned y = 0; y < by; y++)
                for (unsigned x = 0; x < bx; x++) p[x * sx + y * sy + z * sz] = q[16 * z + 4 * y + x];
    }
}

/* ------------------------------------------------------------------------ */
/* ZVC: zero-value compaction (CSWAP+/zfp/compression.cu)                     */
/*                                                                           */
/* The reference runs `process` GPU threads; thread i owns the contiguous    */
/* chunk [E*i, min(E*(i+1), N)) with E = ceil(N/process).  Threads whose      */
/* chunk starts at or past N do nothing.  Here the threads are a serial loop. */
/* ------------------------------------------------------------------------ */

static int ceil_div(int a, int b) { return a / b + (a % b != 0); }

/* elements per chunk (compression.cu:138-142) */
int orc_zvc_chunk_elems(int n, int process) { return ceil_div(n, process); }
/* mask words per chunk (compression.cu:188-192) */
int orc_zvc_chunk_words(int n, int process) { return ceil_div(ceil_div(n, process), 32); }
/* number of chunks that hold data = the scan length the caller passes to
 * PreAcc (Execution.h:90, with exact integer ceilings) */
int orc_zvc_active_chunks(int n, int process) { return ceil_div(n, ceil_div(n, process)); }
/* mask buffer size in bytes (Execution.h:88) */
size_t orc_zvc_mask_bytes(int n, int process)
{
    return (size_t)orc_zvc_chunk_words(n, process) * (size_t)process * sizeof(uint32_t);
}

/* compression.cu:134-165: per-chunk count of elements != 0 (so -0.0 counts as
 * zero and NaN as non-zero).  Entries of chunks without data are untouched. */
void orc_zvc_count(int n, int process, const float *x, int *count)
{
    int E = ceil_div(n, process);
#ifdef _OPENMP
#pragma omp parallel for schedule(static)
#endif
    for (int i = 0; i < process; i++) {
        long long b = (long long)E * i;
        if (b >= n) continue;
        long long e = b + E; if (e > n) e = n;
        int c = 0;
        for (long long k = b; k < e; k++) c += (x[k] != 0);
        count[i] = c;
    }
}

/* compression.cu:9-19: in-place exclusive scan over the first k entries;
 * total goes to *num. */
void orc_zvc_preacc(int *v, int k, int *num)
{
    int run = 0;
    for (int i = 0; i < k; i++) { int c = v[i]; v[i] = run; run += c; }
    *num = run;
}

/* compression.cu:168-239: chunk i appends its non-zeros at values[begin[i]..]
 * and writes ceil(n_i/32) mask words at mask[i*W..], LSB first.  Mask words
 * the reference never writes are left untouched. */
void orc_zvc_compress(int n, int process, const float *x, float *values,
                      const int *begin, uint32_t *mask)
{
    int E = ceil_div(n, process);
    int W = ceil_div(E, 32);
#ifdef _OPENMP
#pragma omp parallel for schedule(static)
#endif
    for (int i = 0; i < process; i++) {
        long long b = (long long)E * i;
        if (b >= n) continue;
        long long e = b + E; if (e > n) e = n;
        int vi = begin[i];
        size_t mi = (size_t)i * W;
        uint32_t acc = 0; int nb = 0;
        for (long long k = b; k < e; k++) {
            if (nb == 32) { mask[mi++] = acc; acc = 0; nb = 0; }
            if (x[k] != 0) { acc |= (uint32_t)1 << nb; values[vi++] = x[k]; }
            nb++;
        }
        mask[mi] = acc;
    }
}

/* Inverse of orc_zvc_compress with the property the reference relies on but
 * does not itself provide (compression.cu:241-318 stops at each word's
 * highest set bit and needs a pre-zeroed destination): every one of the n
 * outputs is written, zeros as +0.0. */
void orc_zvc_decompress(const float *values, const uint32_t *mask, const int *begin,
                        int n, int process, float *out)
{
    int E = ceil_div(n, process);
    int W = ceil_div(E, 32);
#ifdef _OPENMP
#pragma omp parallel for schedule(static)
#endif
    for (int i = 0; i < process; i++) {
        long long b = (long long)E * i;
        if (b >= n) continue;
        long long e = b + E; if (e > n) e = n;
        int vi = begin[i];
        for (long long k = b; k < e; k++) {
            long long r = k - b;
            uint32_t m = mask[(size_t)i * W + (size_t)(r >> 5)];
            out[k] = ((m >> (r & 31)) & 1u) ? values[vi++] : 0.0f;
        }
    }
}

/* The reference kernel exactly as it behaves (compression.cu:241-318): stops
 * at the highest set bit of each mask word, so `out` must be pre-zeroed by the
 * caller for a full reconstruction.  Only defined when n % E == 0. */
void orc_zvc_decompress_reference_writes(const float *values, const uint32_t *mask,
                                         const int *begin, int n, int process, float *out)
{
    int E = ceil_div(n, process);
    int W = ceil_div(E, 32);
    for (int i = 0; i < process; i++) {
        long long b = (long long)E * i;
        if (b >= n) continue;
        int vi = begin[i];
        for (int w = 0; w < W; w++) {
            uint32_t t = mask[(size_t)i * W + w];
            long long k = b + 32LL * w;
            while (t) {
                out[k++] = (t & 1u) ? values[vi++] : 0.0f;
                t >>= 1;
            }
        }
    }
}
