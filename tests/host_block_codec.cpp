// Host build of the product's per-block ZFP codec (cswap_amd/csrc/zfp_block.h),
// so the exact code each GPU lane runs can be compared with the CPU checker
// without a GPU.  Field walking here is deliberately naive.
#include <stddef.h>
#include <string.h>
#include <vector>
#include "../cswap_amd/csrc/zfp_block.h"

namespace {
struct ArraySink {            // ORs block-relative words into the global stream
  uint64_t* words; size_t bit0;
  void put(unsigned j, uint64_t w) {
    size_t p = bit0 + 64 * (size_t)j; size_t i = p >> 6; unsigned s = p & 63;
    words[i] |= w << s;
    if (s) words[i + 1] |= w >> (64 - s);
  }
};
struct ArraySource {
  const uint64_t* words; size_t bit0;
  uint64_t window(unsigned pos) const {
    size_t p = bit0 + pos; size_t i = p >> 6; unsigned s = p & 63;
    uint64_t v = words[i] >> s;
    if (s) v |= words[i + 1] << (64 - s);
    return v;
  }
};
}

extern "C" {

// stream must hold ceil(blocks*maxbits/64)+1 zeroed words
void host_zfp_encode3(const float* in, size_t nx, size_t ny, size_t nz, unsigned maxbits, uint64_t* stream)
{
  size_t mx = (nx + 3) / 4, my = (ny + 3) / 4, mz = (nz + 3) / 4;
  for (size_t b = 0; b < mx * my * mz; b++) {
    size_t x0 = (b % mx) * 4, y0 = ((b / mx) % my) * 4, z0 = (b / (mx * my)) * 4;
    unsigned bx = nx - x0 < 4 ? nx - x0 : 4, by = ny - y0 < 4 ? ny - y0 : 4, bz = nz - z0 < 4 ? nz - z0 : 4;
    float f[64];
    for (int i = 0; i < 64; i++) f[i] = 0.0f;
    for (unsigned z = 0; z < bz; z++) for (unsigned y = 0; y < by; y++) for (unsigned x = 0; x < bx; x++)
      f[x + 4 * y + 16 * z] = in[(x0 + x) + nx * ((y0 + y) + ny * (z0 + z))];
    if (bx < 4 || by < 4 || bz < 4) cswap::pad_block3(f, bx, by, bz);
    ArraySink sink{stream, b * (size_t)maxbits};
    cswap::encode_block(f, maxbits, sink);
  }
}

void host_zfp_decode3(const uint64_t* stream, size_t nx, size_t ny, size_t nz, unsigned maxbits, float* out)
{
  size_t mx = (nx + 3) / 4, my = (ny + 3) / 4, mz = (nz + 3) / 4;
  for (size_t b = 0; b < mx * my * mz; b++) {
    size_t x0 = (b % mx) * 4, y0 = ((b / mx) % my) * 4, z0 = (b / (mx * my)) * 4;
    unsigned bx = nx - x0 < 4 ? nx - x0 : 4, by = ny - y0 < 4 ? ny - y0 : 4, bz = nz - z0 < 4 ? nz - z0 : 4;
    float f[64];
    ArraySource src{stream, b * (size_t)maxbits};
    cswap::decode_block(src, maxbits, f);
    for (unsigned z = 0; z < bz; z++) for (unsigned y = 0; y < by; y++) for (unsigned x = 0; x < bx; x++)
      out[(x0 + x) + nx * ((y0 + y) + ny * (z0 + z))] = f[x + 4 * y + 16 * z];
  }
}

void host_transpose32(uint32_t* a) { uint32_t t[32]; memcpy(t, a, sizeof t); cswap::transpose32(t); memcpy(a, t, sizeof t); }

}
