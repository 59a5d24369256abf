// Host build of the product's per-block ZFP codec (cswap_amd/csrc/zfp_block.h),
// so the exact code each GPU lane runs can be compared with the CPU checker
// without a GPU.  Field walking here is deliberately naive.
#include <stddef.h>
#include <string.h>
#include <vector>
#include "../cswap_amd/csrc/zfp_block.h"

namespace {
struct ArrayBits {            // the bit region is the whole stream, addressed in dwords
  uint32_t* dw;
  void or32(unsigned d, uint32_t v) const { dw[d] |= v; }
  uint32_t ld32(unsigned d) const { return dw[d]; }
};
}

extern "C" {

// stream must hold ceil(blocks*maxbits/64)+2 zeroed words (the codec may touch 96 bits past a block)
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
    ArrayBits mem{reinterpret_cast<uint32_t*>(stream)};
    cswap::encode_block<true>(f, (unsigned)(b * (size_t)maxbits), maxbits, mem);
  }
}

void host_zfp_decode3(const uint64_t* stream, size_t nx, size_t ny, size_t nz, unsigned maxbits, float* out)
{
  size_t mx = (nx + 3) / 4, my = (ny + 3) / 4, mz = (nz + 3) / 4;
  for (size_t b = 0; b < mx * my * mz; b++) {
    size_t x0 = (b % mx) * 4, y0 = ((b / mx) % my) * 4, z0 = (b / (mx * my)) * 4;
    unsigned bx = nx - x0 < 4 ? nx - x0 : 4, by = ny - y0 < 4 ? ny - y0 : 4, bz = nz - z0 < 4 ? nz - z0 : 4;
    float f[64];
    ArrayBits mem{reinterpret_cast<uint32_t*>(const_cast<uint64_t*>(stream))};
    cswap::decode_block(mem, (unsigned)(b * (size_t)maxbits), maxbits, f);
    for (unsigned z = 0; z < bz; z++) for (unsigned y = 0; y < by; y++) for (unsigned x = 0; x < bx; x++)
      out[(x0 + x) + nx * ((y0 + y) + ny * (z0 + z))] = f[x + 4 * y + 16 * z];
  }
}

void host_transpose32(uint32_t* a) { uint32_t t[32]; memcpy(t, a, sizeof t); cswap::transpose32(t); memcpy(a, t, sizeof t); }

}
