// zfp_kernels.hip -- ZFP fixed-rate fp32 3-D encode / decode for gfx950.
//
// Work decomposition: one wavefront (64 lanes) per group of 64 consecutive
// blocks, ONE LANE PER BLOCK.  A lane keeps its 64 coefficients in registers
// through cast, lifting, reorder, bit transpose and the embedded coder
// (zfp_block.h), so there is no cross-lane traffic at all.  The wave's slice of
// the stream (64 blocks x maxbits bits = maxbits 64-bit words, always a whole
// number of words) is staged in LDS, which the coder addresses bit by bit, and
// moved to/from HBM in 16-byte pieces.  Because the stream is fixed-rate,
// stream offsets are closed-form and no device-wide scan, atomic or memset of
// the stream is needed (the reference pre-zeroes the stream and adds every bit
// with a global atomic, CSWAP+/zfp/encode.cuh:252-299, encode3.cuh:152).
#include <hip/hip_runtime.h>
#include <atomic>
#include "../../include/cswap_hip.h"
#include "zfp_block.h"
#include "common.h"

namespace cswap {

struct Field3 {
  uint32_t nx, ny, nz;     // extents in elements
  uint32_t mx, my;         // blocks along x and y
  uint32_t nblocks;
  long long sx, sy, sz;    // strides in elements
  int rows16;              // 1: x-rows of every block are contiguous and 16-byte aligned, rows nest inside
                           //    planes inside the volume, and any 64 consecutive blocks lie within 4 GiB
  int stream16;            // 1: the stream pointer is 16-byte aligned
  int read_once;           // 1: the encoder should load the field with the nontemporal hint (see make_field)
  int once64;              // 1: the decoder of 64-bit elements should store its rows with the hint (see make_field)
  Div31 by_mx, by_my;      // block index -> block coordinates without a hardware divide
};

// Fields of at least this many bytes are loaded with the nontemporal hint (make_field)
#ifndef CSWAP_READ_ONCE_BYTES
#define CSWAP_READ_ONCE_BYTES (128ull << 20)
#endif
constexpr unsigned long long kReadOnceBytes = CSWAP_READ_ONCE_BYTES;

// Fields below this many bytes are coded by the pair form (two wavefronts per 64 blocks)
#ifndef CSWAP_PAIR_ENCODE_BYTES
#define CSWAP_PAIR_ENCODE_BYTES (40ull << 20)
#endif
#ifndef CSWAP_PAIR_DECODE_BYTES
#define CSWAP_PAIR_DECODE_BYTES (40ull << 20)   // and only from 16 bits per value on (kPairDecodeFromBits)
#endif

// 16 bytes of the field as the compiler's own vector type (what the nontemporal builtins take)
typedef float stream_f4 __attribute__((ext_vector_type(4)));
typedef unsigned long long stream_u2 __attribute__((ext_vector_type(2)));

// ------------------------------------------------------------- LDS adapter
// The bit region the block codec ORs into / reads from is LDS: it serves as the
// dynamically indexable extension of the register file (a lane cannot index
// its registers with a run-time bit position).  The codec hands over the byte
// offset of a dword as the LDS address itself, so bit positions count from LDS
// address 0: a block's first bit is bit0 + its offset within the region.  (With
// a pointer to the region plus an offset, every access would cost one more
// instruction that adds the region's address.)
typedef __attribute__((address_space(3))) uint32_t lds_u32;
struct LdsBits {
  unsigned bit0;  // bit position of the region's first bit
  __device__ __forceinline__ explicit LdsBits(uint32_t* region)
      : bit0(8u * (unsigned)(size_t)(__attribute__((address_space(3))) void*)region)
  {
  }
  __device__ __forceinline__ static lds_u32* at(unsigned d) { return (lds_u32*)(size_t)d; }
  __device__ __forceinline__ void or32(unsigned d, uint32_t v) const
  {
    __hip_atomic_fetch_or(at(d), v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);  // ds_or_b32
  }
  __device__ __forceinline__ uint32_t ld32(unsigned d) const { return *at(d); }
};

// Layout of the wave's LDS bit region.
//  whole-word rates (maxbits % 64 == 0): every lane owns a private slot of
//    maxbits + slack bits (slot a multiple of 128 bits), so the coder needs no
//    end-of-block guards and each lane moves its own words to/from HBM;
//  other rates: the 64 blocks are packed back to back exactly as in the stream
//    (always a whole number of words per wave) and moved cooperatively.
__host__ __device__ inline unsigned slot_bits(unsigned maxbits)
{
  return (maxbits & 63u) ? maxbits : ((maxbits + 128u + 127u) & ~127u);
}
__host__ __device__ inline unsigned region_dwords(unsigned maxbits)
{
  return ((2u * slot_bits(maxbits) + 4u) + 3u) & ~3u;  // + padding for the 128-bit over-read / over-write
}
// The 32-bit decoder's slot is the block and its fence of 64 ones, nothing more: the
// window it reads through reaches up to 64 bits further, into the next lane's block
// (or the region's padding), and those bits are never looked at.  What this saves in
// LDS is two more wavefronts per compute unit at 16 bits per value (8720 bytes a
// wavefront instead of 9232), and the stride of 2 (mod 4) dwords halves the bank
// conflicts between lanes.  Slots are 8-byte aligned only.
__host__ __device__ inline unsigned dec_slot_bits(unsigned maxbits)
{
  return (maxbits & 63u) ? maxbits : maxbits + 64u;
}
__host__ __device__ inline unsigned dec_region_dwords(unsigned maxbits)
{
  return ((2u * dec_slot_bits(maxbits) + 4u) + 3u) & ~3u;
}

// ------------------------------------------------------------- block <-> field
__device__ __forceinline__ void block_origin(const Field3& fd, uint32_t b, uint32_t& x0, uint32_t& y0,
                                             uint32_t& z0)
{
  uint32_t q = div31(b, fd.by_mx);
  x0 = (b - q * fd.mx) * 4;
  uint32_t r = div31(q, fd.by_my);
  y0 = (q - r * fd.my) * 4;
  z0 = r * 4;
}

// Addressing of the fast path (Field3::rows16): the wavefront's first block gives
// a wave-uniform 64-bit base, every lane adds a 32-bit byte offset to it.  Block
// order is x, then y, then z and the strides nest, so offsets grow with the block
// index; the host only sets rows16 when 64 consecutive blocks span less than 4 GiB.
struct WaveBase {
  long long origin;  // element offset of the first block's corner
  uint32_t fx, fy, fz;
};
__device__ __forceinline__ WaveBase wave_base(const Field3& fd, uint32_t first)
{
  WaveBase w;
  block_origin(fd, first, w.fx, w.fy, w.fz);
  w.origin = (long long)w.fx + (long long)w.fy * fd.sy + (long long)w.fz * fd.sz;
  return w;
}
__device__ __forceinline__ uint32_t lane_bytes(const Field3& fd, const WaveBase& w, uint32_t x0, uint32_t y0,
                                               uint32_t z0)
{
  return ((x0 - w.fx) + (y0 - w.fy) * (uint32_t)fd.sy + (z0 - w.fz) * (uint32_t)fd.sz) * 4u;  // mod 2^32
}

template <bool ONCE>
__device__ __forceinline__ void load_block(const float* __restrict__ in, const Field3& fd, uint32_t first,
                                           uint32_t b, float (&f)[64])
{
  uint32_t x0, y0, z0;
  block_origin(fd, b, x0, y0, z0);
  uint32_t bx = min(4u, fd.nx - x0), by = min(4u, fd.ny - y0), bz = min(4u, fd.nz - z0);
  if (fd.rows16 && bx == 4 && by == 4 && bz == 4) {
    const WaveBase w = wave_base(fd, first);
    const char* base = reinterpret_cast<const char*>(in + w.origin);
    const uint32_t mine = lane_bytes(fd, w, x0, y0, z0);
    const uint32_t sy4 = (uint32_t)fd.sy * 4u, sz4 = (uint32_t)fd.sz * 4u;
#pragma unroll
    for (int z = 0; z < 4; z++)
#pragma unroll
      for (int y = 0; y < 4; y++) {
        const stream_f4* src = reinterpret_cast<const stream_f4*>(base + (size_t)(mine + (y * sy4 + z * sz4)));
        const stream_f4 v = ONCE ? __builtin_nontemporal_load(src) : *src;
        f[16 * z + 4 * y + 0] = v.x;
        f[16 * z + 4 * y + 1] = v.y;
        f[16 * z + 4 * y + 2] = v.z;
        f[16 * z + 4 * y + 3] = v.w;
      }
  } else {
    const float* p = in + (long long)x0 * fd.sx + (long long)y0 * fd.sy + (long long)z0 * fd.sz;
#pragma unroll
    for (int z = 0; z < 4; z++)
#pragma unroll
      for (int y = 0; y < 4; y++)
#pragma unroll
        for (int x = 0; x < 4; x++) {
          bool ok = (uint32_t)x < bx && (uint32_t)y < by && (uint32_t)z < bz;
          f[16 * z + 4 * y + x] = ok ? p[x * fd.sx + y * fd.sy + z * fd.sz] : 0.0f;
        }
    if (bx < 4 || by < 4 || bz < 4) pad_block3(f, bx, by, bz);
  }
}

// one x-row of an int32 block: last lifting pass, values handed on as bit patterns
__device__ __forceinline__ void decode_row_i32(int32_t (&ib)[64], int row, float (&f)[4])
{
  inv_lift4(ib[4 * row], ib[4 * row + 1], ib[4 * row + 2], ib[4 * row + 3]);
#pragma unroll
  for (int x = 0; x < 4; x++) f[x] = __int_as_float(ib[4 * row + x]);
}

// Finishes the block (inverse lifting along x, cast) and stores it.  Every
// x-row is finished and stored on its own, so the finished values never all
// sit in registers at once.
template <bool INT>
__device__ __forceinline__ void finish_and_store_block(float* __restrict__ out, const Field3& fd, uint32_t first,
                                                       uint32_t b, int32_t (&ib)[64], float w)
{
  uint32_t x0, y0, z0;
  block_origin(fd, b, x0, y0, z0);
  uint32_t bx = min(4u, fd.nx - x0), by = min(4u, fd.ny - y0), bz = min(4u, fd.nz - z0);
  if (fd.rows16 && bx == 4 && by == 4 && bz == 4) {
    const WaveBase wb = wave_base(fd, first);
    char* base = reinterpret_cast<char*>(out + wb.origin);
    const uint32_t mine = lane_bytes(fd, wb, x0, y0, z0);
    const uint32_t sy4 = (uint32_t)fd.sy * 4u, sz4 = (uint32_t)fd.sz * 4u;
#pragma unroll
    for (int z = 0; z < 4; z++)
#pragma unroll
      for (int y = 0; y < 4; y++) {
        float r[4];
        if (INT) decode_row_i32(ib, y + 4 * z, r);
        else decode_row(ib, y + 4 * z, w, r);
        const stream_f4 v = {r[0], r[1], r[2], r[3]};
        __builtin_nontemporal_store(v, reinterpret_cast<stream_f4*>(base + (size_t)(mine + (y * sy4 + z * sz4))));
      }
  } else {
    float* p = out + (long long)x0 * fd.sx + (long long)y0 * fd.sy + (long long)z0 * fd.sz;
#pragma unroll
    for (int z = 0; z < 4; z++)
#pragma unroll
      for (int y = 0; y < 4; y++) {
        float r[4];
        if (INT) decode_row_i32(ib, y + 4 * z, r);
        else decode_row(ib, y + 4 * z, w, r);
#pragma unroll
        for (int x = 0; x < 4; x++)
          if ((uint32_t)x < bx && (uint32_t)y < by && (uint32_t)z < bz) p[x * fd.sx + y * fd.sy + z * fd.sz] = r[x];
      }
  }
}

// ------------------------------------------------------------- LDS region <-> stream
__device__ __forceinline__ void zero_region(uint4* lds_raw, unsigned lane, unsigned maxbits)
{
  const unsigned n16 = region_dwords(maxbits) / 4;
  for (unsigned i = lane; i < n16; i += 64) lds_raw[i] = make_uint4(0, 0, 0, 0);
}

// the wave's coded blocks from LDS to the stream
template <bool WHOLE>
__device__ __forceinline__ void store_region(const uint32_t* lds, unsigned lane, uint32_t first, uint32_t valid,
                                             unsigned maxbits, int stream16, uint64_t* __restrict__ stream)
{
  if (WHOLE) {
    // each lane stores the words of its own block (16-byte stores where aligned)
    if (lane < valid) {
      const unsigned W = maxbits >> 6;
      const uint64_t* src = reinterpret_cast<const uint64_t*>(lds + lane * (slot_bits(maxbits) / 32));
      uint64_t* dst = stream + (size_t)(first + lane) * W;
      if ((W & 1u) == 0 && stream16) {
        for (unsigned j = 0; j < W; j += 2)
          *reinterpret_cast<ulonglong2*>(dst + j) = *reinterpret_cast<const ulonglong2*>(src + j);
      } else {
        for (unsigned j = 0; j < W; j++) dst[j] = src[j];
      }
    }
  } else {
    const unsigned nwords = (valid * maxbits + 63u) >> 6;
    const uint64_t* src = reinterpret_cast<const uint64_t*>(lds);
    uint64_t* dst = stream + (size_t)(first >> 6) * maxbits;
    for (unsigned i = lane; i < nwords; i += 64) dst[i] = src[i];
  }
}

// the wave's coded blocks from the stream into LDS; whole-word rates get the
// fence of ones behind every block that the fenced decoder relies on
template <bool WHOLE, bool SLOT16 = true>
__device__ __forceinline__ void load_region(uint32_t* lds, unsigned lane, uint32_t first, uint32_t valid,
                                            unsigned maxbits, unsigned slot, int stream16,
                                            const uint64_t* __restrict__ stream)
{
  if (WHOLE) {
    if (lane < valid) {
      const unsigned W = maxbits >> 6;
      uint64_t* dst = reinterpret_cast<uint64_t*>(lds + lane * (slot / 32));
      const uint64_t* src = stream + (size_t)(first + lane) * W;
      if ((W & 1u) == 0 && stream16) {
        for (unsigned j = 0; j < W; j += 2) {
          const ulonglong2 v = *reinterpret_cast<const ulonglong2*>(src + j);
          if (SLOT16) {
            *reinterpret_cast<ulonglong2*>(dst + j) = v;
          } else {
            dst[j] = v.x;
            dst[j + 1] = v.y;
          }
        }
      } else {
        for (unsigned j = 0; j < W; j++) dst[j] = src[j];
      }
      dst[W] = ~0ull;
    }
  } else {
    const unsigned nwords = (valid * maxbits + 63u) >> 6;
    const uint64_t* src = stream + (size_t)(first >> 6) * maxbits;
    uint64_t* dst = reinterpret_cast<uint64_t*>(lds);
    for (unsigned i = lane; i < nwords + 2; i += 64) dst[i] = i < nwords ? src[i] : 0;
  }
}

// ------------------------------------------------------------- kernels
// grid.x = ceil(nblocks/64) workgroups of one wavefront; dynamic LDS =
// region_dwords(maxbits) dwords.
// INT: the field holds int32 values (moved as 32-bit patterns through the same loads and stores)
// ONCE: the field is loaded with the nontemporal hint (Field3::read_once)
// WPE: wavefronts per SIMD the kernel is built for and held to.  Five, except from 16 bits
// per value on: there a wavefront's LDS region (9 KB and more) lets 16 or 17 wavefronts
// into a compute unit, unevenly over its SIMDs, and the encoder measured fastest with
// three per SIMD (402.7 MB at 16 bits per value: 130-133 us against 139-140 us with four
// or five), the decoder with four (137-140 us against 143-156 us).
template <bool WHOLE, bool INT = false, bool ONCE = false, int WPE = 5>
__global__ __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(WPE, WPE))) void zfp_encode3_f32_kernel(const float* __restrict__ in, Field3 fd,
                                                             unsigned maxbits,
                                                             uint64_t* __restrict__ stream)
{
  extern __shared__ uint4 lds_raw[];
  uint32_t* lds = reinterpret_cast<uint32_t*>(lds_raw);
  const unsigned lane = threadIdx.x;
  const uint32_t first = blockIdx.x * 64u;
  const uint32_t valid = min(64u, fd.nblocks - first);
  const unsigned slot = slot_bits(maxbits);

  // A wavefront in one of its memory phases (the loads here, the stores at the end) goes before
  // the ones that are coding when both have an instruction to issue: its requests are what the
  // compute unit's other wavefronts will be computing behind (measured on 402.7 MB: encode 100 ->
  // 97 us at 8 bits per value, 129 -> 126 us at 16; the other way round 100 and 131 us).
  float f[64];
  __builtin_amdgcn_s_setprio(3);
  if (lane < valid) load_block<ONCE>(in, fd, first, first + lane, f);  // in flight while the region is cleared
  zero_region(lds_raw, lane, maxbits);
  __syncthreads();
  __builtin_amdgcn_s_setprio(0);

  if (lane < valid) {
    LdsBits mem(lds);
    if (INT) {
      int32_t v[64];
#pragma unroll
      for (int i = 0; i < 64; i++) v[i] = __float_as_int(f[i]);
      encode_block_i32<!WHOLE>(v, mem.bit0 + lane * slot, maxbits, mem);
    } else {
      encode_block<!WHOLE>(f, mem.bit0 + lane * slot, maxbits, mem);
    }
  }
  __syncthreads();
  __builtin_amdgcn_s_setprio(3);
  store_region<WHOLE>(lds, lane, first, valid, maxbits, fd.stream16, stream);
}

// Five wavefronts per SIMD (at most 96 registers, which the row-wise finish
// and the late block coordinates below reach without spilling): measured
// 2.5 % faster than the four that the unconstrained 105 registers allow; six
// (80 registers) spills and is slower again.
template <bool WHOLE, bool INT = false, int WPE = 5>
__global__ __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(WPE, WPE))) void zfp_decode3_f32_kernel(const uint64_t* __restrict__ stream, Field3 fd,
                                                             unsigned maxbits, float* __restrict__ out)
{
  extern __shared__ uint4 lds_raw[];
  uint32_t* lds = reinterpret_cast<uint32_t*>(lds_raw);
  const unsigned lane = threadIdx.x;
  const uint32_t first = blockIdx.x * 64u;
  const uint32_t valid = min(64u, fd.nblocks - first);
  const unsigned slot = dec_slot_bits(maxbits);

  // Issue priorities: the load of the stream and the bit planes (a dependent chain through LDS
  // reads) go first, the lifting along z and y inside decode_block_zy fills the slots that are
  // left, and the last part -- lifting along x, cast, the row stores -- sits between the two.
  // Measured on 402.7 MB: 97.5 us with one priority for everything, 94.3 us with the planes
  // above the rest, 87.8 us with the last part below the planes as well (16 bits per value:
  // 137 -> 129 us); the last part below the lifting: 110 us.
  __builtin_amdgcn_s_setprio(3);
  load_region<WHOLE, false>(lds, lane, first, valid, maxbits, slot, fd.stream16, stream);
  __syncthreads();

  if (lane < valid) {
    int32_t ib[64];
    float w;
    LdsBits mem(lds);
    if (INT) {
      w = 0.0f;
      decode_block_i32_zy<WHOLE>(mem, mem.bit0 + lane * slot, maxbits, ib);
    } else {
      decode_block_zy<WHOLE>(mem, mem.bit0 + lane * slot, maxbits, ib, w);
    }
    // block coordinates and addresses are worked out only now, from a lane id
    // that is recomputed here and tied to a decoded value: otherwise they (or
    // the thread index they come from) are held in registers through the whole
    // decode, or spilled
    uint32_t zero = 0;
    asm volatile("" : "+v"(zero) : "v"(ib[0]));
    const uint32_t b = first + __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, zero));  // lane id again
    __builtin_amdgcn_s_setprio(1);
    finish_and_store_block<INT>(out, fd, first, b, ib, w);
  }
}

// ------------------------------------------------------------- the pair form: two wavefronts per 64 blocks
// For fields that are too small to fill the chip with one lane per block.  A workgroup is two
// wavefronts; lane l of both works on block first + l, each doing its half of every phase
// (zfp_block.h: pair_encode_half), so that a field keeps twice as many wavefronts in flight,
// each with half the serial work.  Fast path only: whole-word rates with an even number of
// 16-byte pieces per block, full blocks, 16-byte aligned contiguous rows.
//
// Dynamic LDS, in dwords: [region: region_dwords(maxbits)] [maxima: 128] [flag: 4]
// [U0: 1280] [U1: 1280].  U0 and U1 carry all three later exchanges in turn, and the rule
// that makes this safe without barriers of its own is that a half only ever writes into the
// one it was the last to read:
//   z exchange   half h writes U_h (lane * 20 + j, four 16-byte pieces)        barrier  reads U_(1-h)
//   reorder      writes the 13 coefficients it sends into U_(1-h) (slot * 64 + lane)
//                                                                               barrier  reads U_h
//   planes       writes its 32 bits of 16 planes into U_h (k * 64 + lane)      barrier  reads both
constexpr unsigned kPairMaxima = 128, kPairFlag = 4, kPairU = 1280;
__host__ __device__ inline unsigned pair_lds_dwords(unsigned maxbits)
{
  return region_dwords(maxbits) + kPairMaxima + kPairFlag + 2 * kPairU;
}

template <int H>
struct LdsExchange {
  float* maxima;
  uint32_t* flag;
  uint32_t* mine;    // U_H
  uint32_t* theirs;  // U_(1-H)
  unsigned lane;
  __device__ __forceinline__ float other_max(float m)
  {
    maxima[H * 64 + lane] = m;
    __syncthreads();
    return maxima[(1 - H) * 64 + lane];
  }
  __device__ __forceinline__ void swap16(const int32_t (&out)[16], int32_t (&in)[16])
  {
    uint4* dst = reinterpret_cast<uint4*>(mine + lane * 20);
#pragma unroll
    for (int j = 0; j < 4; j++)
      dst[j] = make_uint4((uint32_t)out[4 * j], (uint32_t)out[4 * j + 1], (uint32_t)out[4 * j + 2], (uint32_t)out[4 * j + 3]);
    __syncthreads();
    const uint4* src = reinterpret_cast<const uint4*>(theirs + lane * 20);
#pragma unroll
    for (int j = 0; j < 4; j++) {
      const uint4 v = src[j];
      in[4 * j] = (int32_t)v.x;
      in[4 * j + 1] = (int32_t)v.y;
      in[4 * j + 2] = (int32_t)v.z;
      in[4 * j + 3] = (int32_t)v.w;
    }
  }
  __device__ __forceinline__ void seq_put(int slot, uint32_t v) { theirs[slot * 64 + lane] = v; }
  __device__ __forceinline__ void seq_sync() { __syncthreads(); }
  __device__ __forceinline__ uint32_t seq_get(int slot) { return mine[slot * 64 + lane]; }
  __device__ __forceinline__ void plane_put(int k, uint32_t v) { mine[k * 64 + lane] = v; }
  __device__ __forceinline__ void plane_sync() { __syncthreads(); }
  __device__ __forceinline__ uint64_t plane_get(int k)
  {
    const uint32_t* u0 = H == 0 ? mine : theirs;
    const uint32_t* u1 = H == 0 ? theirs : mine;
    return ((uint64_t)u1[k * 64 + lane] << 32) | u0[k * 64 + lane];
  }
  // Half 0 answers for both, so that the two can never disagree about the barriers ahead.
  __device__ __forceinline__ bool more(bool any)
  {
    if (H == 0 && lane == 0) *flag = any ? 1u : 0u;
    __syncthreads();
    return __builtin_amdgcn_readfirstlane(*flag) != 0;
  }
  __device__ __forceinline__ void done() { __syncthreads(); }
};

template <int H>
__device__ __forceinline__ void pair_encode_body(const float* __restrict__ in, const Field3& fd, unsigned maxbits,
                                                 uint32_t* lds, unsigned lane, uint32_t first)
{
  const bool live = first + lane < fd.nblocks;
  const uint32_t b = live ? first + lane : fd.nblocks - 1;
  float p[16], q[16];
  {
    uint32_t x0, y0, z0;
    block_origin(fd, b, x0, y0, z0);
    const WaveBase w = wave_base(fd, first);
    const char* base = reinterpret_cast<const char*>(in + w.origin);
    const uint32_t me = lane_bytes(fd, w, x0, y0, z0);
    const uint32_t sy4 = (uint32_t)fd.sy * 4u, sz4 = (uint32_t)fd.sz * 4u;
    constexpr int ZP = H == 0 ? 0 : 2, ZQ = H == 0 ? 3 : 1;
#pragma unroll
    for (int y = 0; y < 4; y++) {
      const stream_f4 vp = *reinterpret_cast<const stream_f4*>(base + (size_t)(me + (y * sy4 + ZP * sz4)));
      const stream_f4 vq = *reinterpret_cast<const stream_f4*>(base + (size_t)(me + (y * sy4 + ZQ * sz4)));
      p[4 * y] = vp.x; p[4 * y + 1] = vp.y; p[4 * y + 2] = vp.z; p[4 * y + 3] = vp.w;
      q[4 * y] = vq.x; q[4 * y + 1] = vq.y; q[4 * y + 2] = vq.z; q[4 * y + 3] = vq.w;
    }
  }
  const unsigned region = region_dwords(maxbits);
  LdsExchange<H> ex;
  ex.maxima = reinterpret_cast<float*>(lds + region);
  ex.flag = lds + region + kPairMaxima;
  ex.mine = lds + region + kPairMaxima + kPairFlag + H * kPairU;
  ex.theirs = lds + region + kPairMaxima + kPairFlag + (1 - H) * kPairU;
  ex.lane = lane;
  LdsBits mem(lds);
  pair_encode_half<H>(p, q, live, mem.bit0 + lane * slot_bits(maxbits), maxbits, mem, ex);
}

__global__ __launch_bounds__(128) void zfp_encode3_f32_pair_kernel(const float* __restrict__ in, Field3 fd,
                                                                   unsigned maxbits, uint64_t* __restrict__ stream)
{
  extern __shared__ uint4 lds_raw[];
  uint32_t* lds = reinterpret_cast<uint32_t*>(lds_raw);
  const unsigned tid = threadIdx.x, lane = tid & 63u;
  const uint32_t first = blockIdx.x * 64u;
  {  // the region starts out zero; the first exchange's barrier orders this before any coder's OR
    const unsigned n16 = region_dwords(maxbits) / 4;
    for (unsigned i = tid; i < n16; i += 128) lds_raw[i] = make_uint4(0, 0, 0, 0);
  }
  if (__builtin_amdgcn_readfirstlane(tid >> 6) == 0) pair_encode_body<0>(in, fd, maxbits, lds, lane, first);
  else pair_encode_body<1>(in, fd, maxbits, lds, lane, first);
  // Both halves are past the barrier of more() or done(): every block is coded.  Thread t
  // moves half of block t / 2 (W / 2 words, W / 4 16-byte pieces).
  const uint32_t blk = first + (tid >> 1);
  if (blk < fd.nblocks) {
    const unsigned W = maxbits >> 6;
    const ulonglong2* src = reinterpret_cast<const ulonglong2*>(lds + (tid >> 1) * (slot_bits(maxbits) / 32) + (tid & 1u) * W);
    ulonglong2* dst = reinterpret_cast<ulonglong2*>(stream + (size_t)blk * W + (tid & 1u) * (W / 2));
    for (unsigned j = 0; j < W / 4; j++) dst[j] = src[j];
  }
}

// The pair form of the decoder (zfp_block.h: pair_decode_half).  Dynamic LDS, in dwords:
// [region: dec_region_dwords(maxbits)] [scales: 64] [flag: 4] [U0: 1024] [U1: 1024].
//   planes     half 0 writes the low words of 16 plane words into U0 and the high words into U1
//              (k * 64 + lane)                                                barrier  half h reads U_h
//              (the same again for the low 16 planes, between two more barriers, when they follow)
//   reorder    half h writes the 13 coefficients it sends into U_h (slot * 64 + lane)
//                                                                              barrier  reads U_(1-h)
//   z exchange half h writes into U_(1-h) (j * 64 + lane)                     barrier  reads U_h
// again a half only ever writes into the one it was the last to read.
constexpr unsigned kPairScales = 64, kPairDecU = 1024;
__host__ __device__ inline unsigned pair_dec_lds_dwords(unsigned maxbits)
{
  return dec_region_dwords(maxbits) + kPairScales + kPairFlag + 2 * kPairDecU;
}

template <int H>
struct LdsDecExchange {
  float* scales;
  uint32_t* flag;
  uint32_t* u0;
  uint32_t* u1;
  unsigned lane;
  __device__ __forceinline__ uint32_t* mine() const { return H == 0 ? u0 : u1; }
  __device__ __forceinline__ uint32_t* theirs() const { return H == 0 ? u1 : u0; }
  __device__ __forceinline__ void plane_put(int k, uint64_t x)
  {
    u0[k * 64 + lane] = (uint32_t)x;
    u1[k * 64 + lane] = (uint32_t)(x >> 32);
  }
  __device__ __forceinline__ void scale_put(float w) { scales[lane] = w; }
  __device__ __forceinline__ bool planes_sync(bool any)
  {
    if (H == 0 && lane == 0) *flag = any ? 1u : 0u;
    __syncthreads();
    return __builtin_amdgcn_readfirstlane(*flag) != 0;
  }
  __device__ __forceinline__ uint32_t plane_get(int k) { return mine()[k * 64 + lane]; }
  __device__ __forceinline__ float scale_get() { return scales[lane]; }
  __device__ __forceinline__ void consumed() { __syncthreads(); }
  __device__ __forceinline__ void low_sync() { __syncthreads(); }
  __device__ __forceinline__ void seq_put(int slot, uint32_t v) { mine()[slot * 64 + lane] = v; }
  __device__ __forceinline__ void seq_sync() { __syncthreads(); }
  __device__ __forceinline__ uint32_t seq_get(int slot) { return theirs()[slot * 64 + lane]; }
  __device__ __forceinline__ void swap16(const int32_t (&out)[16], int32_t (&in)[16])
  {
#pragma unroll
    for (int j = 0; j < 16; j++) theirs()[j * 64 + lane] = (uint32_t)out[j];
    __syncthreads();
#pragma unroll
    for (int j = 0; j < 16; j++) in[j] = (int32_t)mine()[j * 64 + lane];
  }
};

template <int H>
__device__ __forceinline__ void pair_decode_body(const Field3& fd, unsigned maxbits, uint32_t* lds, unsigned lane,
                                                 uint32_t first, float* __restrict__ out)
{
  const unsigned region = dec_region_dwords(maxbits);
  LdsDecExchange<H> ex;
  ex.scales = reinterpret_cast<float*>(lds + region);
  ex.flag = lds + region + kPairScales;
  ex.u0 = lds + region + kPairScales + kPairFlag;
  ex.u1 = ex.u0 + kPairDecU;
  ex.lane = lane;
  LdsBits mem(lds);
  float p[16], q[16];
  pair_decode_half<H>(mem, mem.bit0 + lane * dec_slot_bits(maxbits), maxbits, ex, p, q);
  if (first + lane < fd.nblocks) {
    uint32_t x0, y0, z0;
    block_origin(fd, first + lane, x0, y0, z0);
    const WaveBase w = wave_base(fd, first);
    char* base = reinterpret_cast<char*>(out + w.origin);
    const uint32_t me = lane_bytes(fd, w, x0, y0, z0);
    const uint32_t sy4 = (uint32_t)fd.sy * 4u, sz4 = (uint32_t)fd.sz * 4u;
    constexpr int ZP = H == 0 ? 0 : 2, ZQ = H == 0 ? 3 : 1;
#pragma unroll
    for (int y = 0; y < 4; y++) {
      const stream_f4 vp = {p[4 * y], p[4 * y + 1], p[4 * y + 2], p[4 * y + 3]};
      const stream_f4 vq = {q[4 * y], q[4 * y + 1], q[4 * y + 2], q[4 * y + 3]};
      __builtin_nontemporal_store(vp, reinterpret_cast<stream_f4*>(base + (size_t)(me + (y * sy4 + ZP * sz4))));
      __builtin_nontemporal_store(vq, reinterpret_cast<stream_f4*>(base + (size_t)(me + (y * sy4 + ZQ * sz4))));
    }
  }
}

__global__ __launch_bounds__(128) void zfp_decode3_f32_pair_kernel(const uint64_t* __restrict__ stream, Field3 fd,
                                                                   unsigned maxbits, float* __restrict__ out)
{
  extern __shared__ uint4 lds_raw[];
  uint32_t* lds = reinterpret_cast<uint32_t*>(lds_raw);
  const unsigned tid = threadIdx.x, lane = tid & 63u;
  const uint32_t first = blockIdx.x * 64u;
  {  // thread t brings in half of block t / 2; the fence of ones behind every block comes with the second half.
     // The slots of blocks past the end of the field read as empty blocks.
    const unsigned W = maxbits >> 6;
    const uint32_t blk = first + (tid >> 1);
    uint64_t* dst = reinterpret_cast<uint64_t*>(lds + (tid >> 1) * (dec_slot_bits(maxbits) / 32)) + (tid & 1u) * (W / 2);
    if (blk < fd.nblocks) {
      const ulonglong2* src = reinterpret_cast<const ulonglong2*>(stream + (size_t)blk * W + (tid & 1u) * (W / 2));
      for (unsigned j = 0; j < W / 4; j++) {
        const ulonglong2 v = src[j];
        dst[2 * j] = v.x;
        dst[2 * j + 1] = v.y;
      }
    } else {
      for (unsigned j = 0; j < W / 2; j++) dst[j] = 0;
    }
    if (tid & 1u) dst[W / 2] = ~0ull;
  }
  __syncthreads();
  if (__builtin_amdgcn_readfirstlane(tid >> 6) == 0) pair_decode_body<0>(fd, maxbits, lds, lane, first, out);
  else pair_decode_body<1>(fd, maxbits, lds, lane, first, out);
}

// ------------------------------------------------------------- 64-bit elements
// Fields of doubles or int64 (zfp_type_double, zfp_type_int64): the same
// decomposition, values moved as 64-bit patterns.  Fast path: full block whose
// x-rows are contiguous and 16-byte aligned (two 16-byte accesses per row).
__device__ __forceinline__ void load_block_w64(const uint64_t* __restrict__ in, const Field3& fd, uint32_t b,
                                               uint64_t (&q)[64])
{
  uint32_t x0, y0, z0;
  block_origin(fd, b, x0, y0, z0);
  const uint32_t bx = min(4u, fd.nx - x0), by = min(4u, fd.ny - y0), bz = min(4u, fd.nz - z0);
  const uint64_t* p = in + (long long)x0 * fd.sx + (long long)y0 * fd.sy + (long long)z0 * fd.sz;
  if (fd.rows16 && bx == 4 && by == 4 && bz == 4) {
#pragma unroll
    for (int z = 0; z < 4; z++)
#pragma unroll
      for (int y = 0; y < 4; y++) {
        const ulonglong2* r = reinterpret_cast<const ulonglong2*>(p + y * fd.sy + z * fd.sz);
        const ulonglong2 a = r[0], c = r[1];
        q[16 * z + 4 * y + 0] = a.x;
        q[16 * z + 4 * y + 1] = a.y;
        q[16 * z + 4 * y + 2] = c.x;
        q[16 * z + 4 * y + 3] = c.y;
      }
  } else {
#pragma unroll
    for (int z = 0; z < 4; z++)
#pragma unroll
      for (int y = 0; y < 4; y++)
#pragma unroll
        for (int x = 0; x < 4; x++) {
          bool ok = (uint32_t)x < bx && (uint32_t)y < by && (uint32_t)z < bz;
          q[16 * z + 4 * y + x] = ok ? p[x * fd.sx + y * fd.sy + z * fd.sz] : 0ull;
        }
    if (bx < 4 || by < 4 || bz < 4) pad_block3(q, bx, by, bz);
  }
}

template <bool ONCE>
__device__ __forceinline__ void store_block_w64(uint64_t* __restrict__ out, const Field3& fd, uint32_t b,
                                                const uint64_t (&q)[64])
{
  uint32_t x0, y0, z0;
  block_origin(fd, b, x0, y0, z0);
  const uint32_t bx = min(4u, fd.nx - x0), by = min(4u, fd.ny - y0), bz = min(4u, fd.nz - z0);
  uint64_t* p = out + (long long)x0 * fd.sx + (long long)y0 * fd.sy + (long long)z0 * fd.sz;
  if (fd.rows16 && bx == 4 && by == 4 && bz == 4) {
#pragma unroll
    for (int z = 0; z < 4; z++)
#pragma unroll
      for (int y = 0; y < 4; y++) {
        stream_u2* r = reinterpret_cast<stream_u2*>(p + y * fd.sy + z * fd.sz);
        const stream_u2 a = {q[16 * z + 4 * y + 0], q[16 * z + 4 * y + 1]};
        const stream_u2 c = {q[16 * z + 4 * y + 2], q[16 * z + 4 * y + 3]};
        if (ONCE) {
          __builtin_nontemporal_store(a, r);
          __builtin_nontemporal_store(c, r + 1);
        } else {
          r[0] = a;
          r[1] = c;
        }
      }
  } else {
#pragma unroll
    for (int z = 0; z < 4; z++)
#pragma unroll
      for (int y = 0; y < 4; y++)
#pragma unroll
        for (int x = 0; x < 4; x++)
          if ((uint32_t)x < bx && (uint32_t)y < by && (uint32_t)z < bz)
            p[x * fd.sx + y * fd.sy + z * fd.sz] = q[16 * z + 4 * y + x];
  }
}

template <bool WHOLE, bool INT>
__global__ __launch_bounds__(64) void zfp_encode3_w64_kernel(const uint64_t* __restrict__ in, Field3 fd,
                                                             unsigned maxbits, uint64_t* __restrict__ stream)
{
  extern __shared__ uint4 lds_raw[];
  uint32_t* lds = reinterpret_cast<uint32_t*>(lds_raw);
  const unsigned lane = threadIdx.x;
  const uint32_t first = blockIdx.x * 64u;
  const uint32_t valid = min(64u, fd.nblocks - first);
  uint64_t q[64];
  if (lane < valid) load_block_w64(in, fd, first + lane, q);  // in flight while the region is cleared
  zero_region(lds_raw, lane, maxbits);
  __syncthreads();
  if (lane < valid) {
    LdsBits mem(lds);
    encode_block_w64<!WHOLE, INT>(q, mem.bit0 + lane * slot_bits(maxbits), maxbits, mem);
  }
  __syncthreads();
  store_region<WHOLE>(lds, lane, first, valid, maxbits, fd.stream16, stream);
}

// ONCE: rows stored with the nontemporal hint (Field3::once64)
template <bool WHOLE, bool INT, bool ONCE = false>
__global__ __launch_bounds__(64) void zfp_decode3_w64_kernel(const uint64_t* __restrict__ stream, Field3 fd,
                                                             unsigned maxbits, uint64_t* __restrict__ out)
{
  extern __shared__ uint4 lds_raw[];
  uint32_t* lds = reinterpret_cast<uint32_t*>(lds_raw);
  const unsigned lane = threadIdx.x;
  const uint32_t first = blockIdx.x * 64u;
  const uint32_t valid = min(64u, fd.nblocks - first);
  __builtin_amdgcn_s_setprio(3);  // the 32-bit decoder's priorities (here, at two wavefronts per SIMD, worth 2.6 %)
  load_region<WHOLE>(lds, lane, first, valid, maxbits, slot_bits(maxbits), fd.stream16, stream);
  __syncthreads();
  if (lane < valid) {
    uint64_t q[64];
    LdsBits mem(lds);
    decode_block_w64<INT, WHOLE>(mem, mem.bit0 + lane * slot_bits(maxbits), maxbits, q);
    __builtin_amdgcn_s_setprio(1);
    store_block_w64<ONCE>(out, fd, first + lane, q);
  }
}

// ------------------------------------------------------------- 2-D / 1-D fields
// Same decomposition (one lane per block of 16 or 4 values, 64 blocks per
// wave, LDS bit region); element accesses are predicated scalars.
struct FieldLow {
  uint32_t nx, ny;   // ny = 1 for a 1-D field
  uint32_t mx;       // blocks along x
  uint32_t nblocks;
  long long sx, sy;
};

template <int DIMS>
__device__ __forceinline__ void load_block_low(const float* __restrict__ in, const FieldLow& fd, uint32_t b,
                                               float (&f)[16])
{
  const uint32_t q = b / fd.mx;
  const uint32_t x0 = (b - q * fd.mx) * 4, y0 = DIMS == 2 ? q * 4 : 0;
  const float* p = in + (long long)x0 * fd.sx + (long long)y0 * fd.sy;
  const uint32_t bx = min(4u, fd.nx - x0), by = DIMS == 2 ? min(4u, fd.ny - y0) : 1u;
#pragma unroll
  for (int y = 0; y < 4; y++)
#pragma unroll
    for (int x = 0; x < 4; x++) {
      bool ok = (uint32_t)x < bx && (uint32_t)y < by;
      f[4 * y + x] = ok ? p[x * fd.sx + y * fd.sy] : 0.0f;
    }
#pragma unroll
  for (int y = 0; y < (DIMS == 2 ? 4 : 1); y++) pad4(f[4 * y], f[4 * y + 1], f[4 * y + 2], f[4 * y + 3], bx);
  if (DIMS == 2) {
#pragma unroll
    for (int x = 0; x < 4; x++) pad4(f[x], f[x + 4], f[x + 8], f[x + 12], by);
  }
}

template <int DIMS>
__device__ __forceinline__ void store_block_low(float* __restrict__ out, const FieldLow& fd, uint32_t b,
                                                const float (&f)[16])
{
  const uint32_t q = b / fd.mx;
  const uint32_t x0 = (b - q * fd.mx) * 4, y0 = DIMS == 2 ? q * 4 : 0;
  float* p = out + (long long)x0 * fd.sx + (long long)y0 * fd.sy;
  const uint32_t bx = min(4u, fd.nx - x0), by = DIMS == 2 ? min(4u, fd.ny - y0) : 1u;
#pragma unroll
  for (int y = 0; y < 4; y++)
#pragma unroll
    for (int x = 0; x < 4; x++)
      if ((uint32_t)x < bx && (uint32_t)y < by) p[x * fd.sx + y * fd.sy] = f[4 * y + x];
}

// The wave's 64 blocks are packed back to back in LDS exactly as in the stream
// (64 * maxbits bits = maxbits whole words) and moved cooperatively.
template <int DIMS, bool INT = false>
__global__ __launch_bounds__(64) void zfp_encode_low_f32_kernel(const float* __restrict__ in, FieldLow fd,
                                                                unsigned maxbits, uint64_t* __restrict__ stream)
{
  extern __shared__ uint4 lds_raw[];
  uint32_t* lds = reinterpret_cast<uint32_t*>(lds_raw);
  const unsigned lane = threadIdx.x;
  const uint32_t first = blockIdx.x * 64u;
  const uint32_t valid = min(64u, fd.nblocks - first);
  const unsigned n16 = (2u * maxbits + 4u + 3u) / 4u;
  for (unsigned i = lane; i < n16; i += 64) lds_raw[i] = make_uint4(0, 0, 0, 0);
  __syncthreads();
  if (lane < valid) {
    float f[16];
    load_block_low<DIMS>(in, fd, first + lane, f);
    LdsBits mem(lds);
    encode_block_low<DIMS, true, INT>(f, mem.bit0 + lane * maxbits, maxbits, mem);
  }
  __syncthreads();
  const unsigned nwords = (valid * maxbits + 63u) >> 6;
  const uint64_t* src = reinterpret_cast<const uint64_t*>(lds);
  uint64_t* dst = stream + (size_t)blockIdx.x * maxbits;
  for (unsigned i = lane; i < nwords; i += 64) dst[i] = src[i];
}

template <int DIMS, bool INT = false>
__global__ __launch_bounds__(64) void zfp_decode_low_f32_kernel(const uint64_t* __restrict__ stream, FieldLow fd,
                                                                unsigned maxbits, float* __restrict__ out)
{
  extern __shared__ uint4 lds_raw[];
  uint32_t* lds = reinterpret_cast<uint32_t*>(lds_raw);
  const unsigned lane = threadIdx.x;
  const uint32_t first = blockIdx.x * 64u;
  const uint32_t valid = min(64u, fd.nblocks - first);
  const unsigned nwords = (valid * maxbits + 63u) >> 6;
  const uint64_t* src = stream + (size_t)blockIdx.x * maxbits;
  uint64_t* dst = reinterpret_cast<uint64_t*>(lds);
  for (unsigned i = lane; i < nwords + 2; i += 64) dst[i] = i < nwords ? src[i] : 0;
  __syncthreads();
  if (lane < valid) {
    float f[16];
    LdsBits mem(lds);
    decode_block_low<DIMS, INT>(mem, mem.bit0 + lane * maxbits, maxbits, f);
    store_block_low<DIMS>(out, fd, first + lane, f);
  }
}

// 64-bit elements, 2-D / 1-D
template <int DIMS, bool INT>
__global__ __launch_bounds__(64) void zfp_encode_low_w64_kernel(const uint64_t* __restrict__ in, FieldLow fd,
                                                                unsigned maxbits, uint64_t* __restrict__ stream)
{
  extern __shared__ uint4 lds_raw[];
  uint32_t* lds = reinterpret_cast<uint32_t*>(lds_raw);
  const unsigned lane = threadIdx.x;
  const uint32_t first = blockIdx.x * 64u;
  const uint32_t valid = min(64u, fd.nblocks - first);
  const unsigned n16 = (2u * maxbits + 4u + 3u) / 4u;
  for (unsigned i = lane; i < n16; i += 64) lds_raw[i] = make_uint4(0, 0, 0, 0);
  __syncthreads();
  if (lane < valid) {
    const uint32_t b = first + lane;
    const uint32_t r = b / fd.mx;
    const uint32_t x0 = (b - r * fd.mx) * 4, y0 = DIMS == 2 ? r * 4 : 0;
    const uint64_t* p = in + (long long)x0 * fd.sx + (long long)y0 * fd.sy;
    const uint32_t bx = min(4u, fd.nx - x0), by = DIMS == 2 ? min(4u, fd.ny - y0) : 1u;
    uint64_t q[16];
#pragma unroll
    for (int y = 0; y < 4; y++)
#pragma unroll
      for (int x = 0; x < 4; x++) {
        bool ok = (uint32_t)x < bx && (uint32_t)y < by;
        q[4 * y + x] = ok ? p[x * fd.sx + y * fd.sy] : 0ull;
      }
#pragma unroll
    for (int y = 0; y < (DIMS == 2 ? 4 : 1); y++) pad4(q[4 * y], q[4 * y + 1], q[4 * y + 2], q[4 * y + 3], bx);
    if (DIMS == 2) {
#pragma unroll
      for (int x = 0; x < 4; x++) pad4(q[x], q[x + 4], q[x + 8], q[x + 12], by);
    }
    LdsBits mem(lds);
    encode_block_low_w64<DIMS, true, INT>(q, mem.bit0 + lane * maxbits, maxbits, mem);
  }
  __syncthreads();
  const unsigned nwords = (valid * maxbits + 63u) >> 6;
  const uint64_t* src = reinterpret_cast<const uint64_t*>(lds);
  uint64_t* dst = stream + (size_t)blockIdx.x * maxbits;
  for (unsigned i = lane; i < nwords; i += 64) dst[i] = src[i];
}

template <int DIMS, bool INT>
__global__ __launch_bounds__(64) void zfp_decode_low_w64_kernel(const uint64_t* __restrict__ stream, FieldLow fd,
                                                                unsigned maxbits, uint64_t* __restrict__ out)
{
  extern __shared__ uint4 lds_raw[];
  uint32_t* lds = reinterpret_cast<uint32_t*>(lds_raw);
  const unsigned lane = threadIdx.x;
  const uint32_t first = blockIdx.x * 64u;
  const uint32_t valid = min(64u, fd.nblocks - first);
  const unsigned nwords = (valid * maxbits + 63u) >> 6;
  const uint64_t* src = stream + (size_t)blockIdx.x * maxbits;
  uint64_t* dst = reinterpret_cast<uint64_t*>(lds);
  for (unsigned i = lane; i < nwords + 2; i += 64) dst[i] = i < nwords ? src[i] : 0;
  __syncthreads();
  if (lane < valid) {
    uint64_t q[16];
    LdsBits mem(lds);
    decode_block_low_w64<DIMS, INT>(mem, mem.bit0 + lane * maxbits, maxbits, q);
    const uint32_t b = first + lane;
    const uint32_t r = b / fd.mx;
    const uint32_t x0 = (b - r * fd.mx) * 4, y0 = DIMS == 2 ? r * 4 : 0;
    uint64_t* p = out + (long long)x0 * fd.sx + (long long)y0 * fd.sy;
    const uint32_t bx = min(4u, fd.nx - x0), by = DIMS == 2 ? min(4u, fd.ny - y0) : 1u;
#pragma unroll
    for (int y = 0; y < 4; y++)
#pragma unroll
      for (int x = 0; x < 4; x++)
        if ((uint32_t)x < bx && (uint32_t)y < by) p[x * fd.sx + y * fd.sy] = q[4 * y + x];
  }
}

static int make_field_low(FieldLow& fd, int dims, const void* base, const void* stream, size_t nx, size_t ny,
                          ptrdiff_t sx, ptrdiff_t sy, unsigned maxbits, unsigned elem)
{
  if (dims == 1) ny = 1;
  if (!nx || !ny || maxbits < 16 || maxbits > 4096) return CSWAP_E_ARG;
  if (nx > 0x7fffffffu || ny > 0x7fffffffu) return CSWAP_E_ARG;
  if (((uintptr_t)stream % 8) != 0 || ((uintptr_t)base % elem) != 0) return CSWAP_E_ARG;
  size_t mx = (nx + 3) / 4, my = dims == 2 ? (ny + 3) / 4 : 1;
  size_t nb = mx * my;
  if (nb > 0xfffffff0ull) return CSWAP_E_ARG;
  fd.nx = (uint32_t)nx; fd.ny = (uint32_t)ny; fd.mx = (uint32_t)mx; fd.nblocks = (uint32_t)nb;
  fd.sx = sx ? sx : 1;
  fd.sy = sy ? sy : (ptrdiff_t)nx;
  return CSWAP_OK;
}

// ------------------------------------------------------------- host side
static int make_field(Field3& fd, const void* base, const void* stream, size_t nx, size_t ny, size_t nz,
                      ptrdiff_t sx, ptrdiff_t sy, ptrdiff_t sz, unsigned maxbits, unsigned elem)
{
  if (((uintptr_t)stream % 8) != 0 || ((uintptr_t)base % elem) != 0) return CSWAP_E_ARG;
  if (!nx || !ny || !nz) return CSWAP_E_ARG;
  if (maxbits < 16 || maxbits > 4096) return CSWAP_E_ARG;
  if (nx > 0x7fffffffu || ny > 0x7fffffffu || nz > 0x7fffffffu) return CSWAP_E_ARG;
  size_t mx = (nx + 3) / 4, my = (ny + 3) / 4, mz = (nz + 3) / 4;
  size_t nb = mx * my * mz;
  if (nb / mz != mx * my || nb > 0x7fffffffull) return CSWAP_E_ARG;  // block indices stay below 2^31
  fd.nx = (uint32_t)nx; fd.ny = (uint32_t)ny; fd.nz = (uint32_t)nz;
  fd.mx = (uint32_t)mx; fd.my = (uint32_t)my;
  fd.nblocks = (uint32_t)nb;
  fd.sx = sx ? sx : 1;
  fd.sy = sy ? sy : (ptrdiff_t)nx;
  fd.sz = sz ? sz : (ptrdiff_t)(nx * ny);
  fd.by_mx = make_div31(fd.mx);
  fd.by_my = make_div31(fd.my);
  // fast path: aligned contiguous rows; rows inside planes inside the volume (so
  // element offsets grow with the block index); and the slabs of four planes that
  // 64 consecutive blocks can touch (one more than they fill) stay below 4 GiB, so
  // every block of a wavefront is within a 32-bit byte offset of its first block
  const size_t slabs = (64 + mx * my - 1) / (mx * my) + 1;
  const ptrdiff_t per16 = (ptrdiff_t)(16 / elem);  // elements in 16 bytes
  fd.rows16 = fd.sx == 1 && (fd.sy % per16) == 0 && (fd.sz % per16) == 0 && ((uintptr_t)base % 16) == 0 &&
              fd.sy >= (ptrdiff_t)nx && fd.sz >= fd.sy * (ptrdiff_t)ny &&
              (unsigned long long)fd.sz * 4ull * elem * slabs < 0xfff00000ull;
  fd.stream16 = ((uintptr_t)stream % 16) == 0;
  // Cache policy of the field's 16-byte rows (whole 128-byte lines per wave instruction).
  // The decoder always stores them with the nontemporal hint: 402.7 MB decode in 107 us
  // instead of 117 us, and the kernel that runs next no longer waits behind those lines
  // draining from the memory-side cache (33.6 MB: decode 14.5 instead of 17.6 us, and a
  // reader of the result right after it is no slower).  The encoder loads with the hint
  // only when the field is large against that cache (256 MB): a smaller tensor is still
  // cached from the kernel that produced it, and hinted loads of cached lines are slower.
  // Producer kernel + encoder, hinted / plain loads: 402.7 MB 205 / 220 us, 201.3 MB
  // 95 / 109 us, 100.7 MB 43.6 / 43.2 us, 50.3 MB 26.1 / 24.5 us.  The stream keeps the
  // default policy: a lane's piece of it is not a whole line, and the decoder or the copy
  // engine reads it next.
  fd.read_once = (unsigned long long)nx * ny * nz * elem >= kReadOnceBytes;
  // 64-bit elements: a lane's row is two 16-byte pieces, half a line per store instruction.  The
  // hint on those stores gains 15 % at 537 MB and loses 20 % at 134 MB: only for fields of 256 MiB
  // and more (the memory-side cache's size).
  fd.once64 = elem == 8 && (unsigned long long)nx * ny * nz * elem >= (256ull << 20);
  return CSWAP_OK;
}

}  // namespace cswap

using namespace cswap;

extern "C" size_t cswap_zfp_stream_bytes(size_t nx, size_t ny, size_t nz, unsigned maxbits)
{
  size_t nb = ((nx + 3) / 4) * ((ny + 3) / 4) * ((nz + 3) / 4);
  return (nb * maxbits / 64) * 8;
}

extern "C" size_t cswap_zfp_stream_capacity(size_t nx, size_t ny, size_t nz, unsigned maxbits)
{
  size_t nb = ((nx + 3) / 4) * ((ny + 3) / 4) * ((nz + 3) / 4);
  return ((nb * maxbits + 63) / 64) * 8;
}

// element kinds of a field
enum Elem { kF32 = 0, kI32 = 1, kF64 = 2, kI64 = 3 };
// whole-word rates from this many bits per block of 64 values on run the 32-bit kernels built for fewer wavefronts per SIMD
constexpr unsigned kFewerWavesFrom = 1024;
static unsigned elem_bytes(Elem e) { return e == kF32 || e == kI32 ? 4u : 8u; }

// Fields below this many bytes are coded by the pair form where their shape allows
// (cswap_zfp_set_pair_bytes).
static std::atomic<unsigned long long> g_pair_encode_bytes{CSWAP_PAIR_ENCODE_BYTES};

// what the pair kernels take: the fast path of the field (aligned contiguous rows, an aligned
// stream), full blocks only, and a whole-word rate whose blocks split into two halves of
// whole 16-byte pieces
static bool pair_shape(const Field3& fd, unsigned maxbits)
{
  return fd.rows16 && fd.stream16 && (maxbits & 255u) == 0 && ((fd.nx | fd.ny | fd.nz) & 3u) == 0;
}

static std::atomic<unsigned long long> g_pair_decode_bytes{CSWAP_PAIR_DECODE_BYTES};

// The pair form pays while all of a field's workgroups are on the chip at once (twice the
// wavefronts, each with half the serial work); a field that needs a second round of them is
// faster with one lane per block.  How many workgroups a compute unit holds is set by their
// LDS: measured, 88 % of what its 160 KB divided by the workgroup's bytes allows.  A limit of
// SIZE_MAX takes the form for every field it can code (tests, measurements).
static bool pair_fits(unsigned grid, size_t lds_bytes, unsigned long long limit)
{
  if (limit == ~0ull) return true;
  const double per_cu = 0.88 * 160.0 * 1024.0 / (double)lds_bytes;
  return (double)grid <= per_cu * (double)device_compute_units();
}
// The decoder's pair form gains nothing at 8 bits per value (the plane loop, which one half
// runs alone, is 60 % of its time) and 3-7 % from 16 bits per value on, where the shared back
// end weighs more.
constexpr unsigned kPairDecodeFromBits = 1024;

extern "C" void cswap_zfp_set_pair_bytes(size_t encode_below, size_t decode_below, size_t* previous)
{
  const size_t e = (size_t)g_pair_encode_bytes.exchange(encode_below, std::memory_order_relaxed);
  const size_t d = (size_t)g_pair_decode_bytes.exchange(decode_below, std::memory_order_relaxed);
  if (previous) {
    previous[0] = e;
    previous[1] = d;
  }
}

#define CSWAP_LAUNCH3(KERNEL_, T_, ARG0_, ARG3_)                                                                   \
  do {                                                                                                              \
    if (whole && !is_int)                                                                                           \
      hipLaunchKernelGGL((KERNEL_<true, false>), dim3(grid), dim3(64), lds_bytes, st, ARG0_, fd, maxbits, ARG3_);   \
    else if (!whole && !is_int)                                                                                     \
      hipLaunchKernelGGL((KERNEL_<false, false>), dim3(grid), dim3(64), lds_bytes, st, ARG0_, fd, maxbits, ARG3_);  \
    else if (whole)                                                                                                 \
      hipLaunchKernelGGL((KERNEL_<true, true>), dim3(grid), dim3(64), lds_bytes, st, ARG0_, fd, maxbits, ARG3_);    \
    else                                                                                                            \
      hipLaunchKernelGGL((KERNEL_<false, true>), dim3(grid), dim3(64), lds_bytes, st, ARG0_, fd, maxbits, ARG3_);   \
  } while (0)

static int compress3(const void* d_in, Elem elem, size_t nx, size_t ny, size_t nz, ptrdiff_t sx, ptrdiff_t sy,
                     ptrdiff_t sz, unsigned maxbits, uint64_t* d_stream, cswap_stream_t stream)
{
  if (!d_in || !d_stream) return CSWAP_E_ARG;
  Field3 fd;
  int rc = make_field(fd, d_in, d_stream, nx, ny, nz, sx, sy, sz, maxbits, elem_bytes(elem));
  if (rc) return rc;
  unsigned grid = (fd.nblocks + 63) / 64;
  size_t lds_bytes = (size_t)region_dwords(maxbits) * 4;
  hipStream_t st = (hipStream_t)stream;
  const bool whole = (maxbits & 63u) == 0;
  const bool is_int = elem == kI32 || elem == kI64;
  const unsigned long long pair_below = g_pair_encode_bytes.load(std::memory_order_relaxed);
  if (elem == kF32 && pair_shape(fd, maxbits) && (unsigned long long)nx * ny * nz * 4ull < pair_below &&
      pair_fits(grid, (size_t)pair_lds_dwords(maxbits) * 4, pair_below)) {
    hipLaunchKernelGGL(zfp_encode3_f32_pair_kernel, dim3(grid), dim3(128), (size_t)pair_lds_dwords(maxbits) * 4, st,
                       static_cast<const float*>(d_in), fd, maxbits, d_stream);
    return check_launch();
  }
  if (elem_bytes(elem) == 4) {
    const float* in = static_cast<const float*>(d_in);
    const bool once = fd.read_once && fd.rows16;
    if (whole && maxbits >= kFewerWavesFrom) {
      if (once && !is_int)
        hipLaunchKernelGGL((zfp_encode3_f32_kernel<true, false, true, 3>), dim3(grid), dim3(64), lds_bytes, st, in,
                           fd, maxbits, d_stream);
      else if (once)
        hipLaunchKernelGGL((zfp_encode3_f32_kernel<true, true, true, 3>), dim3(grid), dim3(64), lds_bytes, st, in,
                           fd, maxbits, d_stream);
      else if (!is_int)
        hipLaunchKernelGGL((zfp_encode3_f32_kernel<true, false, false, 3>), dim3(grid), dim3(64), lds_bytes, st, in,
                           fd, maxbits, d_stream);
      else
        hipLaunchKernelGGL((zfp_encode3_f32_kernel<true, true, false, 3>), dim3(grid), dim3(64), lds_bytes, st, in,
                           fd, maxbits, d_stream);
    } else if (fd.read_once && fd.rows16 && whole && !is_int)
      hipLaunchKernelGGL((zfp_encode3_f32_kernel<true, false, true>), dim3(grid), dim3(64), lds_bytes, st, in, fd,
                         maxbits, d_stream);
    else if (fd.read_once && fd.rows16 && whole)
      hipLaunchKernelGGL((zfp_encode3_f32_kernel<true, true, true>), dim3(grid), dim3(64), lds_bytes, st, in, fd,
                         maxbits, d_stream);
    else
      CSWAP_LAUNCH3(zfp_encode3_f32_kernel, float, in, d_stream);
  } else {
    const uint64_t* in = static_cast<const uint64_t*>(d_in);
    CSWAP_LAUNCH3(zfp_encode3_w64_kernel, uint64_t, in, d_stream);
  }
  return check_launch();
}

static int decompress3(const uint64_t* d_stream, Elem elem, size_t nx, size_t ny, size_t nz, ptrdiff_t sx,
                       ptrdiff_t sy, ptrdiff_t sz, unsigned maxbits, void* d_out, cswap_stream_t stream)
{
  if (!d_out || !d_stream) return CSWAP_E_ARG;
  Field3 fd;
  int rc = make_field(fd, d_out, d_stream, nx, ny, nz, sx, sy, sz, maxbits, elem_bytes(elem));
  if (rc) return rc;
  unsigned grid = (fd.nblocks + 63) / 64;
  size_t lds_bytes = (size_t)region_dwords(maxbits) * 4;
  hipStream_t st = (hipStream_t)stream;
  const bool whole = (maxbits & 63u) == 0;
  const bool is_int = elem == kI32 || elem == kI64;
  const unsigned long long pair_below = g_pair_decode_bytes.load(std::memory_order_relaxed);
  if (elem == kF32 && pair_shape(fd, maxbits) && (unsigned long long)nx * ny * nz * 4ull < pair_below &&
      (maxbits >= kPairDecodeFromBits || pair_below == ~0ull) &&
      pair_fits(grid, (size_t)pair_dec_lds_dwords(maxbits) * 4, pair_below)) {
    hipLaunchKernelGGL(zfp_decode3_f32_pair_kernel, dim3(grid), dim3(128), (size_t)pair_dec_lds_dwords(maxbits) * 4, st,
                       d_stream, fd, maxbits, static_cast<float*>(d_out));
    return check_launch();
  }
  if (elem_bytes(elem) == 4) {
    float* out = static_cast<float*>(d_out);
    lds_bytes = (size_t)dec_region_dwords(maxbits) * 4;
    if (whole && maxbits >= kFewerWavesFrom && !is_int)
      hipLaunchKernelGGL((zfp_decode3_f32_kernel<true, false, 4>), dim3(grid), dim3(64), lds_bytes, st, d_stream, fd,
                         maxbits, out);
    else if (whole && maxbits >= kFewerWavesFrom)
      hipLaunchKernelGGL((zfp_decode3_f32_kernel<true, true, 4>), dim3(grid), dim3(64), lds_bytes, st, d_stream, fd,
                         maxbits, out);
    else
      CSWAP_LAUNCH3(zfp_decode3_f32_kernel, float, d_stream, out);
  } else {
    uint64_t* out = static_cast<uint64_t*>(d_out);
    if (fd.once64 && fd.rows16 && whole && !is_int)
      hipLaunchKernelGGL((zfp_decode3_w64_kernel<true, false, true>), dim3(grid), dim3(64), lds_bytes, st, d_stream,
                         fd, maxbits, out);
    else if (fd.once64 && fd.rows16 && whole)
      hipLaunchKernelGGL((zfp_decode3_w64_kernel<true, true, true>), dim3(grid), dim3(64), lds_bytes, st, d_stream,
                         fd, maxbits, out);
    else
      CSWAP_LAUNCH3(zfp_decode3_w64_kernel, uint64_t, d_stream, out);
  }
  return check_launch();
}
#undef CSWAP_LAUNCH3

extern "C" int cswap_zfp_compress_f32(const float* d_in, size_t nx, size_t ny, size_t nz, ptrdiff_t sx,
                                      ptrdiff_t sy, ptrdiff_t sz, unsigned maxbits, uint64_t* d_stream,
                                      cswap_stream_t stream)
{
  return compress3(d_in, kF32, nx, ny, nz, sx, sy, sz, maxbits, d_stream, stream);
}

extern "C" int cswap_zfp_decompress_f32(const uint64_t* d_stream, size_t nx, size_t ny, size_t nz,
                                        ptrdiff_t sx, ptrdiff_t sy, ptrdiff_t sz, unsigned maxbits,
                                        float* d_out, cswap_stream_t stream)
{
  return decompress3(d_stream, kF32, nx, ny, nz, sx, sy, sz, maxbits, d_out, stream);
}

// ------------------------------------------------------------- any dimensionality
static size_t blocks_nd(int dims, size_t nx, size_t ny, size_t nz)
{
  size_t nb = (nx + 3) / 4;
  if (dims >= 2) nb *= (ny + 3) / 4;
  if (dims >= 3) nb *= (nz + 3) / 4;
  return nb;
}

extern "C" size_t cswap_zfp_stream_capacity_nd(int dims, size_t nx, size_t ny, size_t nz, unsigned maxbits)
{
  if (dims < 1 || dims > 3) return 0;
  return ((blocks_nd(dims, nx, ny, nz) * maxbits + 63) / 64) * 8;
}

extern "C" size_t cswap_zfp_stream_bytes_nd(int dims, size_t nx, size_t ny, size_t nz, unsigned maxbits)
{
  if (dims < 1 || dims > 3) return 0;
  if (dims == 3) return cswap_zfp_stream_bytes(nx, ny, nz, maxbits);
  return cswap_zfp_stream_capacity_nd(dims, nx, ny, nz, maxbits);  // 1-D and 2-D round up (zfp/shared.h:42-71)
}

#define CSWAP_LAUNCH_LOW(KERNEL_, ARG0_, ARG3_)                                                                  \
  do {                                                                                                             \
    if (dims == 2 && !is_int)                                                                                      \
      hipLaunchKernelGGL((KERNEL_<2, false>), dim3(grid), dim3(64), lds_bytes, st, ARG0_, fd, maxbits, ARG3_);     \
    else if (dims == 2)                                                                                            \
      hipLaunchKernelGGL((KERNEL_<2, true>), dim3(grid), dim3(64), lds_bytes, st, ARG0_, fd, maxbits, ARG3_);      \
    else if (!is_int)                                                                                              \
      hipLaunchKernelGGL((KERNEL_<1, false>), dim3(grid), dim3(64), lds_bytes, st, ARG0_, fd, maxbits, ARG3_);     \
    else                                                                                                           \
      hipLaunchKernelGGL((KERNEL_<1, true>), dim3(grid), dim3(64), lds_bytes, st, ARG0_, fd, maxbits, ARG3_);      \
  } while (0)

static int compress_nd(const void* d_in, Elem elem, int dims, size_t nx, size_t ny, size_t nz, ptrdiff_t sx,
                       ptrdiff_t sy, ptrdiff_t sz, unsigned maxbits, uint64_t* d_stream, cswap_stream_t stream)
{
  if (dims == 3) return compress3(d_in, elem, nx, ny, nz, sx, sy, sz, maxbits, d_stream, stream);
  if (!d_in || !d_stream || (dims != 1 && dims != 2)) return CSWAP_E_ARG;
  FieldLow fd;
  int rc = make_field_low(fd, dims, d_in, d_stream, nx, ny, sx, sy, maxbits, elem_bytes(elem));
  if (rc) return rc;
  unsigned grid = (fd.nblocks + 63) / 64;
  size_t lds_bytes = (size_t)((2u * maxbits + 4u + 3u) / 4u) * 16;
  hipStream_t st = (hipStream_t)stream;
  const bool is_int = elem == kI32 || elem == kI64;
  if (elem_bytes(elem) == 4) {
    const float* in = static_cast<const float*>(d_in);
    CSWAP_LAUNCH_LOW(zfp_encode_low_f32_kernel, in, d_stream);
  } else {
    const uint64_t* in = static_cast<const uint64_t*>(d_in);
    CSWAP_LAUNCH_LOW(zfp_encode_low_w64_kernel, in, d_stream);
  }
  return check_launch();
}

static int decompress_nd(const uint64_t* d_stream, Elem elem, int dims, size_t nx, size_t ny, size_t nz,
                         ptrdiff_t sx, ptrdiff_t sy, ptrdiff_t sz, unsigned maxbits, void* d_out,
                         cswap_stream_t stream)
{
  if (dims == 3) return decompress3(d_stream, elem, nx, ny, nz, sx, sy, sz, maxbits, d_out, stream);
  if (!d_out || !d_stream || (dims != 1 && dims != 2)) return CSWAP_E_ARG;
  FieldLow fd;
  int rc = make_field_low(fd, dims, d_out, d_stream, nx, ny, sx, sy, maxbits, elem_bytes(elem));
  if (rc) return rc;
  unsigned grid = (fd.nblocks + 63) / 64;
  size_t lds_bytes = (size_t)((2u * maxbits + 4u + 3u) / 4u) * 16;
  hipStream_t st = (hipStream_t)stream;
  const bool is_int = elem == kI32 || elem == kI64;
  if (elem_bytes(elem) == 4) {
    float* out = static_cast<float*>(d_out);
    CSWAP_LAUNCH_LOW(zfp_decode_low_f32_kernel, d_stream, out);
  } else {
    uint64_t* out = static_cast<uint64_t*>(d_out);
    CSWAP_LAUNCH_LOW(zfp_decode_low_w64_kernel, d_stream, out);
  }
  return check_launch();
}
#undef CSWAP_LAUNCH_LOW

extern "C" int cswap_zfp_compress_f32_nd(const float* d_in, int dims, size_t nx, size_t ny, size_t nz, ptrdiff_t sx,
                                         ptrdiff_t sy, ptrdiff_t sz, unsigned maxbits, uint64_t* d_stream,
                                         cswap_stream_t stream)
{
  return compress_nd(d_in, kF32, dims, nx, ny, nz, sx, sy, sz, maxbits, d_stream, stream);
}

extern "C" int cswap_zfp_decompress_f32_nd(const uint64_t* d_stream, int dims, size_t nx, size_t ny, size_t nz,
                                           ptrdiff_t sx, ptrdiff_t sy, ptrdiff_t sz, unsigned maxbits, float* d_out,
                                           cswap_stream_t stream)
{
  return decompress_nd(d_stream, kF32, dims, nx, ny, nz, sx, sy, sz, maxbits, d_out, stream);
}

extern "C" int cswap_zfp_compress_i32_nd(const int32_t* d_in, int dims, size_t nx, size_t ny, size_t nz, ptrdiff_t sx,
                                         ptrdiff_t sy, ptrdiff_t sz, unsigned maxbits, uint64_t* d_stream,
                                         cswap_stream_t stream)
{
  return compress_nd(d_in, kI32, dims, nx, ny, nz, sx, sy, sz, maxbits, d_stream, stream);
}

extern "C" int cswap_zfp_decompress_i32_nd(const uint64_t* d_stream, int dims, size_t nx, size_t ny, size_t nz,
                                           ptrdiff_t sx, ptrdiff_t sy, ptrdiff_t sz, unsigned maxbits,
                                           int32_t* d_out, cswap_stream_t stream)
{
  return decompress_nd(d_stream, kI32, dims, nx, ny, nz, sx, sy, sz, maxbits, d_out, stream);
}

extern "C" int cswap_zfp_compress_f64_nd(const double* d_in, int dims, size_t nx, size_t ny, size_t nz, ptrdiff_t sx,
                                         ptrdiff_t sy, ptrdiff_t sz, unsigned maxbits, uint64_t* d_stream,
                                         cswap_stream_t stream)
{
  return compress_nd(d_in, kF64, dims, nx, ny, nz, sx, sy, sz, maxbits, d_stream, stream);
}

extern "C" int cswap_zfp_decompress_f64_nd(const uint64_t* d_stream, int dims, size_t nx, size_t ny, size_t nz,
                                           ptrdiff_t sx, ptrdiff_t sy, ptrdiff_t sz, unsigned maxbits, double* d_out,
                                           cswap_stream_t stream)
{
  return decompress_nd(d_stream, kF64, dims, nx, ny, nz, sx, sy, sz, maxbits, d_out, stream);
}

extern "C" int cswap_zfp_compress_i64_nd(const int64_t* d_in, int dims, size_t nx, size_t ny, size_t nz, ptrdiff_t sx,
                                         ptrdiff_t sy, ptrdiff_t sz, unsigned maxbits, uint64_t* d_stream,
                                         cswap_stream_t stream)
{
  return compress_nd(d_in, kI64, dims, nx, ny, nz, sx, sy, sz, maxbits, d_stream, stream);
}

extern "C" int cswap_zfp_decompress_i64_nd(const uint64_t* d_stream, int dims, size_t nx, size_t ny, size_t nz,
                                           ptrdiff_t sx, ptrdiff_t sy, ptrdiff_t sz, unsigned maxbits,
                                           int64_t* d_out, cswap_stream_t stream)
{
  return decompress_nd(d_stream, kI64, dims, nx, ny, nz, sx, sy, sz, maxbits, d_out, stream);
}
