// Host build of the product's per-block ZFP codec (cswap_amd/csrc/zfp_block.h),
// so the exact code each GPU lane runs can be compared with the CPU checker
// without a GPU.  Field walking here is deliberately naive.
#include <pthread.h>
#include <stddef.h>
#include <string.h>
#include <vector>
#include "../cswap_amd/csrc/zfp_block.h"

namespace {
struct ArrayBits {            // the bit region is the whole stream, addressed by the byte offset of a dword
  uint32_t* dw;
  void or32(unsigned d, uint32_t v) const { dw[d / 4] |= v; }
  uint32_t ld32(unsigned d) const { return dw[d / 4]; }
};
struct WatchedBits {          // the same for reading, remembering the highest dword that was asked for
  const uint32_t* dw;
  unsigned* top;
  uint32_t ld32(unsigned d) const
  {
    if (d / 4 > *top) *top = d / 4;
    return dw[d / 4];
  }
};
}

extern "C" {

// stream must hold ceil(blocks*maxbits/64)+2 zeroed words (the codec may touch 128 bits past a block)
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

// Same encode through the unguarded variant: every block is coded into a private,
// zeroed slot of maxbits + 128 bits, as the device does for whole-word rates, and
// only its first maxbits bits are kept.  Returns the highest dword index (relative
// to the slot) that any block wrote a non-zero value to.
unsigned host_zfp_encode3_slots(const float* in, size_t nx, size_t ny, size_t nz, unsigned maxbits, uint64_t* stream)
{
  size_t mx = (nx + 3) / 4, my = (ny + 3) / 4, mz = (nz + 3) / 4;
  const unsigned W = maxbits / 64;  // maxbits % 64 == 0
  const unsigned slot_dwords = 2 * W + 4 + 8;  // 8 more so that a write past the 128 bits of slack is seen, not a crash
  uint32_t* slot = new uint32_t[slot_dwords];
  unsigned top = 0;
  for (size_t b = 0; b < mx * my * mz; b++) {
    size_t x0 = (b % mx) * 4, y0 = ((b / mx) % my) * 4, z0 = (b / (mx * my)) * 4;
    unsigned bx = nx - x0 < 4 ? nx - x0 : 4, by = ny - y0 < 4 ? ny - y0 : 4, bz = nz - z0 < 4 ? nz - z0 : 4;
    float f[64];
    for (int i = 0; i < 64; i++) f[i] = 0.0f;
    for (unsigned z = 0; z < bz; z++) for (unsigned y = 0; y < by; y++) for (unsigned x = 0; x < bx; x++)
      f[x + 4 * y + 16 * z] = in[(x0 + x) + nx * ((y0 + y) + ny * (z0 + z))];
    if (bx < 4 || by < 4 || bz < 4) cswap::pad_block3(f, bx, by, bz);
    memset(slot, 0, 4 * (size_t)slot_dwords);
    ArrayBits mem{slot};
    cswap::encode_block<false>(f, 0u, maxbits, mem);
    memcpy(stream + b * W, slot, 8 * (size_t)W);
    for (unsigned d = 0; d < slot_dwords; d++) if (slot[d] && d > top) top = d;
  }
  delete[] slot;
  return top;
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

// Same decode through the fenced variant: every block is copied into a private
// slot that is followed by 64 one bits, as the device does for whole-word rates,
// and then by whatever the next lane's slot happens to hold (here: `junk`,
// different for every block).  Returns the highest dword index, relative to the
// slot, that any block read.
unsigned host_zfp_decode3_fenced(const uint64_t* stream, size_t nx, size_t ny, size_t nz, unsigned maxbits, float* out,
                                 uint32_t junk)
{
  size_t mx = (nx + 3) / 4, my = (ny + 3) / 4, mz = (nz + 3) / 4;
  const unsigned W = maxbits / 64;  // maxbits % 64 == 0
  uint32_t* slot = new uint32_t[2 * W + 16];
  unsigned top = 0;
  for (size_t b = 0; b < mx * my * mz; b++) {
    size_t x0 = (b % mx) * 4, y0 = ((b / mx) % my) * 4, z0 = (b / (mx * my)) * 4;
    unsigned bx = nx - x0 < 4 ? nx - x0 : 4, by = ny - y0 < 4 ? ny - y0 : 4, bz = nz - z0 < 4 ? nz - z0 : 4;
    memcpy(slot, stream + b * W, 8 * (size_t)W);
    slot[2 * W] = slot[2 * W + 1] = 0xffffffffu;
    for (unsigned d = 2 * W + 2; d < 2 * W + 16; d++) slot[d] = junk = junk * 1664525u + 1013904223u + (uint32_t)b;
    float f[64];
    WatchedBits mem{slot, &top};
    cswap::decode_block<true>(mem, 0u, maxbits, f);
    for (unsigned z = 0; z < bz; z++) for (unsigned y = 0; y < by; y++) for (unsigned x = 0; x < bx; x++)
      out[(x0 + x) + nx * ((y0 + y) + ny * (z0 + z))] = f[x + 4 * y + 16 * z];
  }
  delete[] slot;
  return top;
}

// 2-D field a[ny][nx] (ny = 0: 1-D field a[nx])
void host_zfp_encode_low(const float* in, size_t nx, size_t ny, unsigned maxbits, uint64_t* stream)
{
  const int dims = ny ? 2 : 1;
  size_t mx = (nx + 3) / 4, my = ny ? (ny + 3) / 4 : 1;
  for (size_t b = 0; b < mx * my; b++) {
    size_t x0 = (b % mx) * 4, y0 = (b / mx) * 4;
    unsigned bx = nx - x0 < 4 ? nx - x0 : 4, by = dims == 2 ? (ny - y0 < 4 ? ny - y0 : 4) : 1;
    float f[16];
    for (int i = 0; i < 16; i++) f[i] = 0.0f;
    for (unsigned y = 0; y < by; y++) for (unsigned x = 0; x < bx; x++) f[x + 4 * y] = in[(x0 + x) + nx * (y0 + y)];
    for (unsigned y = 0; y < (dims == 2 ? 4u : 1u); y++) cswap::pad4(f[4 * y], f[4 * y + 1], f[4 * y + 2], f[4 * y + 3], bx);
    if (dims == 2) for (int x = 0; x < 4; x++) cswap::pad4(f[x], f[x + 4], f[x + 8], f[x + 12], by);
    ArrayBits mem{reinterpret_cast<uint32_t*>(stream)};
    if (dims == 2) cswap::encode_block_low<2, true>(f, (unsigned)(b * (size_t)maxbits), maxbits, mem);
    else cswap::encode_block_low<1, true>(f, (unsigned)(b * (size_t)maxbits), maxbits, mem);
  }
}

void host_zfp_decode_low(const uint64_t* stream, size_t nx, size_t ny, unsigned maxbits, float* out)
{
  const int dims = ny ? 2 : 1;
  size_t mx = (nx + 3) / 4, my = ny ? (ny + 3) / 4 : 1;
  for (size_t b = 0; b < mx * my; b++) {
    size_t x0 = (b % mx) * 4, y0 = (b / mx) * 4;
    unsigned bx = nx - x0 < 4 ? nx - x0 : 4, by = dims == 2 ? (ny - y0 < 4 ? ny - y0 : 4) : 1;
    float f[16];
    ArrayBits mem{reinterpret_cast<uint32_t*>(const_cast<uint64_t*>(stream))};
    if (dims == 2) cswap::decode_block_low<2>(mem, (unsigned)(b * (size_t)maxbits), maxbits, f);
    else cswap::decode_block_low<1>(mem, (unsigned)(b * (size_t)maxbits), maxbits, f);
    for (unsigned y = 0; y < by; y++) for (unsigned x = 0; x < bx; x++) out[(x0 + x) + nx * (y0 + y)] = f[x + 4 * y];
  }
}

// int32 fields through the same header: dims = 1, 2 or 3, contiguous a[nz][ny][nx]
static void gather_i32(const int32_t* in, int dims, size_t nx, size_t ny, size_t nz, size_t b, float* f, unsigned& bx,
                       unsigned& by, unsigned& bz, size_t& x0, size_t& y0, size_t& z0)
{
  size_t mx = (nx + 3) / 4, my = dims >= 2 ? (ny + 3) / 4 : 1;
  x0 = (b % mx) * 4; y0 = ((b / mx) % my) * 4; z0 = (b / (mx * my)) * 4;
  bx = nx - x0 < 4 ? nx - x0 : 4;
  by = dims >= 2 ? (ny - y0 < 4 ? ny - y0 : 4) : 1;
  bz = dims >= 3 ? (nz - z0 < 4 ? nz - z0 : 4) : 1;
  for (int i = 0; i < 64; i++) f[i] = 0.0f;
  for (unsigned z = 0; z < bz; z++) for (unsigned y = 0; y < by; y++) for (unsigned x = 0; x < bx; x++) {
    int32_t v = in[(x0 + x) + nx * ((y0 + y) + ny * (z0 + z))];
    memcpy(&f[x + 4 * y + 16 * z], &v, 4);
  }
}

void host_zfp_encode_i32(const int32_t* in, int dims, size_t nx, size_t ny, size_t nz, unsigned maxbits, uint64_t* stream)
{
  if (dims < 2) ny = 1;
  if (dims < 3) nz = 1;
  size_t blocks = ((nx + 3) / 4) * (dims >= 2 ? (ny + 3) / 4 : 1) * (dims >= 3 ? (nz + 3) / 4 : 1);
  for (size_t b = 0; b < blocks; b++) {
    float f[64];
    unsigned bx, by, bz; size_t x0, y0, z0;
    gather_i32(in, dims, nx, ny, nz, b, f, bx, by, bz, x0, y0, z0);
    ArrayBits mem{reinterpret_cast<uint32_t*>(stream)};
    if (dims == 3) {
      if (bx < 4 || by < 4 || bz < 4) cswap::pad_block3(f, bx, by, bz);
      int32_t v[64];
      memcpy(v, f, sizeof v);
      cswap::encode_block_i32<true>(v, (unsigned)(b * (size_t)maxbits), maxbits, mem);
    } else {
      float g[16];
      for (int i = 0; i < 16; i++) g[i] = f[i];
      for (int y = 0; y < (dims == 2 ? 4 : 1); y++) cswap::pad4(g[4 * y], g[4 * y + 1], g[4 * y + 2], g[4 * y + 3], bx);
      if (dims == 2) {
        for (int x = 0; x < 4; x++) cswap::pad4(g[x], g[x + 4], g[x + 8], g[x + 12], by);
        cswap::encode_block_low<2, true, true>(g, (unsigned)(b * (size_t)maxbits), maxbits, mem);
      } else {
        cswap::encode_block_low<1, true, true>(g, (unsigned)(b * (size_t)maxbits), maxbits, mem);
      }
    }
  }
}

void host_zfp_decode_i32(const uint64_t* stream, int dims, size_t nx, size_t ny, size_t nz, unsigned maxbits, int32_t* out)
{
  if (dims < 2) ny = 1;
  if (dims < 3) nz = 1;
  size_t mx = (nx + 3) / 4, my = dims >= 2 ? (ny + 3) / 4 : 1, mz = dims >= 3 ? (nz + 3) / 4 : 1;
  for (size_t b = 0; b < mx * my * mz; b++) {
    size_t x0 = (b % mx) * 4, y0 = ((b / mx) % my) * 4, z0 = (b / (mx * my)) * 4;
    unsigned bx = nx - x0 < 4 ? nx - x0 : 4, by = dims >= 2 ? (ny - y0 < 4 ? ny - y0 : 4) : 1,
             bz = dims >= 3 ? (nz - z0 < 4 ? nz - z0 : 4) : 1;
    int32_t v[64];
    ArrayBits mem{reinterpret_cast<uint32_t*>(const_cast<uint64_t*>(stream))};
    if (dims == 3) {
      cswap::decode_block_i32(mem, (unsigned)(b * (size_t)maxbits), maxbits, v);
    } else {
      float g[16];
      if (dims == 2) cswap::decode_block_low<2, true>(mem, (unsigned)(b * (size_t)maxbits), maxbits, g);
      else cswap::decode_block_low<1, true>(mem, (unsigned)(b * (size_t)maxbits), maxbits, g);
      for (int i = 0; i < 64; i++) v[i] = 0;
      memcpy(v, g, sizeof g);
    }
    for (unsigned z = 0; z < bz; z++) for (unsigned y = 0; y < by; y++) for (unsigned x = 0; x < bx; x++)
      out[(x0 + x) + nx * ((y0 + y) + ny * (z0 + z))] = v[x + 4 * y + 16 * z];
  }
}

uint32_t host_div31(uint32_t b, uint32_t d) { return cswap::div31(b, cswap::make_div31(d)); }

float host_decode_scale(uint32_t e8) { return cswap::decode_scale(e8); }

void host_transpose32(uint32_t* a) { uint32_t t[32]; memcpy(t, a, sizeof t); cswap::transpose32(t); memcpy(a, t, sizeof t); }


// 64-bit element types: in / out are 64-bit patterns of doubles (is_int 0) or int64 (is_int 1);
// dims 1..3, a[nz][ny][nx] contiguous
void host_zfp_encode_w64(const uint64_t* in, int is_int, int dims, size_t nx, size_t ny, size_t nz, unsigned maxbits,
                         uint64_t* stream)
{
  if (dims < 2) ny = 1;
  if (dims < 3) nz = 1;
  size_t mx = (nx + 3) / 4, my = dims >= 2 ? (ny + 3) / 4 : 1, mz = dims >= 3 ? (nz + 3) / 4 : 1;
  for (size_t b = 0; b < mx * my * mz; b++) {
    size_t x0 = (b % mx) * 4, y0 = ((b / mx) % my) * 4, z0 = (b / (mx * my)) * 4;
    unsigned bx = nx - x0 < 4 ? nx - x0 : 4, by = dims >= 2 ? (ny - y0 < 4 ? ny - y0 : 4) : 1,
             bz = dims >= 3 ? (nz - z0 < 4 ? nz - z0 : 4) : 1;
    uint64_t q[64];
    for (int i = 0; i < 64; i++) q[i] = 0;
    for (unsigned z = 0; z < bz; z++) for (unsigned y = 0; y < by; y++) for (unsigned x = 0; x < bx; x++)
      q[x + 4 * y + 16 * z] = in[(x0 + x) + nx * ((y0 + y) + ny * (z0 + z))];
    ArrayBits mem{reinterpret_cast<uint32_t*>(stream)};
    const unsigned pos = (unsigned)(b * (size_t)maxbits);
    if (dims == 3) {
      if (bx < 4 || by < 4 || bz < 4) cswap::pad_block3(q, bx, by, bz);
      if (is_int) cswap::encode_block_w64<true, true>(q, pos, maxbits, mem);
      else cswap::encode_block_w64<true, false>(q, pos, maxbits, mem);
    } else {
      uint64_t r[16];
      for (int i = 0; i < 16; i++) r[i] = q[i];
      for (int y = 0; y < (dims == 2 ? 4 : 1); y++) cswap::pad4(r[4 * y], r[4 * y + 1], r[4 * y + 2], r[4 * y + 3], bx);
      if (dims == 2)
        for (int x = 0; x < 4; x++) cswap::pad4(r[x], r[x + 4], r[x + 8], r[x + 12], by);
      if (dims == 2 && is_int) cswap::encode_block_low_w64<2, true, true>(r, pos, maxbits, mem);
      else if (dims == 2) cswap::encode_block_low_w64<2, true, false>(r, pos, maxbits, mem);
      else if (is_int) cswap::encode_block_low_w64<1, true, true>(r, pos, maxbits, mem);
      else cswap::encode_block_low_w64<1, true, false>(r, pos, maxbits, mem);
    }
  }
}

void host_zfp_decode_w64(const uint64_t* stream, int is_int, int dims, size_t nx, size_t ny, size_t nz,
                         unsigned maxbits, uint64_t* out)
{
  if (dims < 2) ny = 1;
  if (dims < 3) nz = 1;
  size_t mx = (nx + 3) / 4, my = dims >= 2 ? (ny + 3) / 4 : 1, mz = dims >= 3 ? (nz + 3) / 4 : 1;
  for (size_t b = 0; b < mx * my * mz; b++) {
    size_t x0 = (b % mx) * 4, y0 = ((b / mx) % my) * 4, z0 = (b / (mx * my)) * 4;
    unsigned bx = nx - x0 < 4 ? nx - x0 : 4, by = dims >= 2 ? (ny - y0 < 4 ? ny - y0 : 4) : 1,
             bz = dims >= 3 ? (nz - z0 < 4 ? nz - z0 : 4) : 1;
    uint64_t q[64];
    for (int i = 0; i < 64; i++) q[i] = 0;
    ArrayBits mem{reinterpret_cast<uint32_t*>(const_cast<uint64_t*>(stream))};
    const unsigned pos = (unsigned)(b * (size_t)maxbits);
    if (dims == 3) {
      if (is_int) cswap::decode_block_w64<true>(mem, pos, maxbits, q);
      else cswap::decode_block_w64<false>(mem, pos, maxbits, q);
    } else {
      uint64_t r[16];
      if (dims == 2 && is_int) cswap::decode_block_low_w64<2, true>(mem, pos, maxbits, r);
      else if (dims == 2) cswap::decode_block_low_w64<2, false>(mem, pos, maxbits, r);
      else if (is_int) cswap::decode_block_low_w64<1, true>(mem, pos, maxbits, r);
      else cswap::decode_block_low_w64<1, false>(mem, pos, maxbits, r);
      for (int i = 0; i < 16; i++) q[i] = r[i];
    }
    for (unsigned z = 0; z < bz; z++) for (unsigned y = 0; y < by; y++) for (unsigned x = 0; x < bx; x++)
      out[(x0 + x) + nx * ((y0 + y) + ny * (z0 + z))] = q[x + 4 * y + 16 * z];
  }
}

}

// ---- the encoder's pair form (a block shared by two wavefronts): two host threads stand for
// the two halves, a thread barrier for the workgroup barrier, and the shared words are laid
// out and reused exactly as the kernel reuses its LDS (a half writes what it sends for the
// reorder over what it has just read of the z exchange, and its plane words over what it has
// just read of the reorder), so a step that overwrote something the partner still needs, or a
// barrier one half takes and the other does not, shows up here: as a wrong stream or as a
// test that never ends.
namespace {
struct AtomicBits {
  uint32_t* dw;
  void or32(unsigned d, uint32_t v) const { __atomic_fetch_or(&dw[d / 4], v, __ATOMIC_RELAXED); }
  uint32_t ld32(unsigned d) const { return dw[d / 4]; }
};
struct PairShared {
  float mx[2];
  uint32_t u[2][16];
  int flag;
  pthread_barrier_t bar;
};
template <int H>
struct HostExchange {
  PairShared& sh;
  void wait() { pthread_barrier_wait(&sh.bar); }
  float other_max(float m) { sh.mx[H] = m; wait(); return sh.mx[1 - H]; }
  void swap16(const int32_t (&out)[16], int32_t (&in)[16])
  {
    for (int i = 0; i < 16; i++) sh.u[H][i] = (uint32_t)out[i];
    wait();
    for (int i = 0; i < 16; i++) in[i] = (int32_t)sh.u[1 - H][i];
  }
  void seq_put(int slot, uint32_t v) { sh.u[1 - H][slot] = v; }
  void seq_sync() { wait(); }
  uint32_t seq_get(int slot) { return sh.u[H][slot]; }
  void plane_put(int k, uint32_t v) { sh.u[H][k] = v; }
  void plane_sync() { wait(); }
  uint64_t plane_get(int k) { return ((uint64_t)sh.u[1][k] << 32) | sh.u[0][k]; }
  bool more(bool mine) { if (H == 0) sh.flag = mine; wait(); return sh.flag != 0; }
  void done() { wait(); }
};
struct PairJob {
  const float* in; size_t nx, ny, nz; unsigned maxbits; uint32_t* slots; unsigned slot_dwords; PairShared* sh;
};
template <int H>
void* pair_thread(void* arg)
{
  PairJob& j = *static_cast<PairJob*>(arg);
  const size_t mx = j.nx / 4, my = j.ny / 4, mz = j.nz / 4;
  HostExchange<H> ex{*j.sh};
  for (size_t b = 0; b < mx * my * mz; b++) {
    const size_t x0 = (b % mx) * 4, y0 = ((b / mx) % my) * 4, z0 = (b / (mx * my)) * 4;
    const int zp = H == 0 ? 0 : 2, zq = H == 0 ? 3 : 1;
    float p[16], q[16];
    for (int y = 0; y < 4; y++) for (int x = 0; x < 4; x++) {
      p[x + 4 * y] = j.in[(x0 + x) + j.nx * ((y0 + y) + j.ny * (z0 + zp))];
      q[x + 4 * y] = j.in[(x0 + x) + j.nx * ((y0 + y) + j.ny * (z0 + zq))];
    }
    AtomicBits mem{j.slots + b * j.slot_dwords};
    cswap::pair_encode_half<H>(p, q, true, 0u, j.maxbits, mem, ex);
  }
  return nullptr;
}
}

extern "C" {
// nx, ny, nz multiples of 4; maxbits a multiple of 64.  Returns the highest dword index
// (relative to its slot) that any block wrote a non-zero value to, or ~0u on a setup error.
unsigned host_zfp_encode3_pair(const float* in, size_t nx, size_t ny, size_t nz, unsigned maxbits, uint64_t* stream)
{
  if (nx % 4 || ny % 4 || nz % 4 || maxbits % 64) return ~0u;
  const size_t nb = (nx / 4) * (ny / 4) * (nz / 4);
  const unsigned W = maxbits / 64, slot_dwords = 2 * W + 4 + 8;
  std::vector<uint32_t> slots(nb * slot_dwords, 0u);
  PairShared sh;
  memset(&sh, 0, sizeof sh);
  if (pthread_barrier_init(&sh.bar, nullptr, 2)) return ~0u;
  PairJob job{in, nx, ny, nz, maxbits, slots.data(), slot_dwords, &sh};
  pthread_t t0, t1;
  pthread_create(&t0, nullptr, pair_thread<0>, &job);
  pthread_create(&t1, nullptr, pair_thread<1>, &job);
  pthread_join(t0, nullptr);
  pthread_join(t1, nullptr);
  pthread_barrier_destroy(&sh.bar);
  unsigned top = 0;
  for (size_t b = 0; b < nb; b++) {
    memcpy(stream + b * W, slots.data() + b * slot_dwords, 8 * (size_t)W);
    for (unsigned d = 0; d < slot_dwords; d++) if (slots[b * slot_dwords + d] && d > top) top = d;
  }
  return top;
}

// BlockEncoder::skip_plane against BlockEncoder::plane on one plane: starting from n known
// coefficients (acc = their mask) at bit position pos of a zeroed region, returns 1 if both
// leave the same n and pos.
int host_skip_plane_agrees(uint64_t x, unsigned n, unsigned pos, unsigned maxbits)
{
  uint32_t region[64];
  memset(region, 0, sizeof region);
  ArrayBits mem{region};
  cswap::BlockEncoder<ArrayBits, false> a(mem, 0u, maxbits), b(mem, 0u, maxbits);
  a.pos = b.pos = pos;
  a.n = b.n = n;
  uint64_t acc = n >= 64 ? ~0ull : (n ? ((~0ull) >> (64 - n)) : 0ull);  // any mask whose highest one-bit is n - 1 does
  if (n) acc = 1ull << (n - 1);
  a.plane(x);
  b.skip_plane(x, acc);
  return a.n == b.n && a.pos == b.pos;
}
}

// ---- the decoder's pair form, the same way: two threads, the kernel's reuse of its shared words
namespace {
struct PairDecShared {
  float scale;
  uint32_t u[2][16];
  int flag;
  pthread_barrier_t bar;
};
template <int H>
struct HostDecExchange {
  PairDecShared& sh;
  void wait() { pthread_barrier_wait(&sh.bar); }
  void plane_put(int k, uint64_t x) { sh.u[0][k] = (uint32_t)x; sh.u[1][k] = (uint32_t)(x >> 32); }
  void scale_put(float w) { sh.scale = w; }
  bool planes_sync(bool any) { if (H == 0) sh.flag = any; wait(); return sh.flag != 0; }
  uint32_t plane_get(int k) { return sh.u[H][k]; }
  float scale_get() { return sh.scale; }
  void consumed() { wait(); }
  void low_sync() { wait(); }
  void seq_put(int slot, uint32_t v) { sh.u[H][slot] = v; }
  void seq_sync() { wait(); }
  uint32_t seq_get(int slot) { return sh.u[1 - H][slot]; }
  void swap16(const int32_t (&out)[16], int32_t (&in)[16])
  {
    for (int j = 0; j < 16; j++) sh.u[1 - H][j] = (uint32_t)out[j];
    wait();
    for (int j = 0; j < 16; j++) in[j] = (int32_t)sh.u[H][j];
  }
};
struct PairDecJob {
  const uint32_t* slots; unsigned slot_dwords; size_t nx, ny, nz; unsigned maxbits; float* out; PairDecShared* sh;
};
template <int H>
void* pair_dec_thread(void* arg)
{
  PairDecJob& j = *static_cast<PairDecJob*>(arg);
  const size_t mx = j.nx / 4, my = j.ny / 4, mz = j.nz / 4;
  HostDecExchange<H> ex{*j.sh};
  for (size_t b = 0; b < mx * my * mz; b++) {
    const size_t x0 = (b % mx) * 4, y0 = ((b / mx) % my) * 4, z0 = (b / (mx * my)) * 4;
    const int zp = H == 0 ? 0 : 2, zq = H == 0 ? 3 : 1;
    ArrayBits mem{const_cast<uint32_t*>(j.slots + b * j.slot_dwords)};
    float p[16], q[16];
    cswap::pair_decode_half<H>(mem, 0u, j.maxbits, ex, p, q);
    for (int y = 0; y < 4; y++) for (int x = 0; x < 4; x++) {
      j.out[(x0 + x) + j.nx * ((y0 + y) + j.ny * (z0 + zp))] = p[x + 4 * y];
      j.out[(x0 + x) + j.nx * ((y0 + y) + j.ny * (z0 + zq))] = q[x + 4 * y];
    }
    ex.wait();  // the shared words are reused by the next block
  }
  return nullptr;
}
}

extern "C" int host_zfp_decode3_pair(const uint64_t* stream, size_t nx, size_t ny, size_t nz, unsigned maxbits, float* out)
{
  if (nx % 4 || ny % 4 || nz % 4 || maxbits % 64) return -1;
  const size_t nb = (nx / 4) * (ny / 4) * (nz / 4);
  const unsigned W = maxbits / 64, slot_dwords = 2 * W + 16;
  std::vector<uint32_t> slots(nb * slot_dwords);
  uint32_t junk = 12345u;
  for (size_t b = 0; b < nb; b++) {  // the block, its fence of 64 ones, then whatever
    uint32_t* s = slots.data() + b * slot_dwords;
    memcpy(s, stream + b * W, 8 * (size_t)W);
    s[2 * W] = s[2 * W + 1] = 0xffffffffu;
    for (unsigned d = 2 * W + 2; d < slot_dwords; d++) s[d] = junk = junk * 1664525u + 1013904223u;
  }
  PairDecShared sh;
  memset(&sh, 0, sizeof sh);
  if (pthread_barrier_init(&sh.bar, nullptr, 2)) return -1;
  PairDecJob job{slots.data(), slot_dwords, nx, ny, nz, maxbits, out, &sh};
  pthread_t t0, t1;
  pthread_create(&t0, nullptr, pair_dec_thread<0>, &job);
  pthread_create(&t1, nullptr, pair_dec_thread<1>, &job);
  pthread_join(t0, nullptr);
  pthread_join(t1, nullptr);
  pthread_barrier_destroy(&sh.bar);
  return 0;
}
