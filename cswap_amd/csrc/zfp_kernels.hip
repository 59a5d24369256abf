// zfp_kernels.hip -- ZFP fixed-rate fp32 3-D encode / decode for gfx950.
//
// Work decomposition: one wavefront (64 lanes) per group of 64 consecutive
// blocks, ONE LANE PER BLOCK.  A lane keeps its 64 coefficients in registers
// through cast, lifting, reorder, bit transpose and the embedded coder
// (zfp_block.h), so there is no cross-lane traffic at all.  The wave's slice of
// the stream (64 blocks x maxbits bits = maxbits 64-bit words, always a whole
// number of words) is staged in LDS in its final layout and moved to/from HBM
// with fully coalesced 8-byte accesses.  Because the stream is fixed-rate,
// stream offsets are closed-form and no device-wide scan, atomic or memset of
// the stream is needed (the reference pre-zeroes the stream and adds every bit
// with a global atomic, CSWAP+/zfp/encode.cuh:252-299, encode3.cuh:152).
#include <hip/hip_runtime.h>
#include "../../include/cswap_hip.h"
#include "zfp_block.h"
#include "common.h"

namespace cswap {

struct Field3 {
  uint32_t nx, ny, nz;     // extents in elements
  uint32_t mx, my;         // blocks along x and y
  uint32_t nblocks;
  long long sx, sy, sz;    // strides in elements
  int rows16;              // 1: x-rows of every block are contiguous, 16-byte aligned
};

// ------------------------------------------------------------- LDS adapters
struct LdsSink {
  uint64_t* lds;
  unsigned bit0;     // first bit of this lane's block inside the wave's slice
  bool whole_words;  // maxbits % 64 == 0: the block owns its words outright
  __device__ __forceinline__ void put(unsigned j, uint64_t w)
  {
    unsigned p = bit0 + 64 * j;
    unsigned i = p >> 6, s = p & 63;
    if (whole_words) {
      lds[i] = w;
    } else {
      atomicOr((unsigned long long*)&lds[i], (unsigned long long)(w << s));
      if (s) atomicOr((unsigned long long*)&lds[i + 1], (unsigned long long)(w >> (64 - s)));
    }
  }
};

struct LdsSource {
  const uint64_t* lds;
  unsigned bit0;
  __device__ __forceinline__ uint64_t window(unsigned pos) const
  {
    unsigned p = bit0 + pos;
    unsigned i = p >> 6, s = p & 63;
    uint64_t lo = lds[i], hi = lds[i + 1];
    return (lo >> s) | ((hi << 1) << (63 - s));
  }
};

// ------------------------------------------------------------- block <-> field
__device__ __forceinline__ void block_origin(const Field3& fd, uint32_t b, uint32_t& x0, uint32_t& y0,
                                             uint32_t& z0)
{
  uint32_t q = b / fd.mx;
  x0 = (b - q * fd.mx) * 4;
  uint32_t r = q / fd.my;
  y0 = (q - r * fd.my) * 4;
  z0 = r * 4;
}

__device__ __forceinline__ void load_block(const float* __restrict__ in, const Field3& fd, uint32_t b,
                                           float (&f)[64])
{
  uint32_t x0, y0, z0;
  block_origin(fd, b, x0, y0, z0);
  const float* p = in + (long long)x0 * fd.sx + (long long)y0 * fd.sy + (long long)z0 * fd.sz;
  uint32_t bx = min(4u, fd.nx - x0), by = min(4u, fd.ny - y0), bz = min(4u, fd.nz - z0);
  if (fd.rows16 && bx == 4 && by == 4 && bz == 4) {
#pragma unroll
    for (int z = 0; z < 4; z++)
#pragma unroll
      for (int y = 0; y < 4; y++) {
        float4 v = *reinterpret_cast<const float4*>(p + y * fd.sy + z * fd.sz);
        f[16 * z + 4 * y + 0] = v.x;
        f[16 * z + 4 * y + 1] = v.y;
        f[16 * z + 4 * y + 2] = v.z;
        f[16 * z + 4 * y + 3] = v.w;
      }
  } else {
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

__device__ __forceinline__ void store_block(float* __restrict__ out, const Field3& fd, uint32_t b,
                                            const float (&f)[64])
{
  uint32_t x0, y0, z0;
  block_origin(fd, b, x0, y0, z0);
  float* p = out + (long long)x0 * fd.sx + (long long)y0 * fd.sy + (long long)z0 * fd.sz;
  uint32_t bx = min(4u, fd.nx - x0), by = min(4u, fd.ny - y0), bz = min(4u, fd.nz - z0);
  if (fd.rows16 && bx == 4 && by == 4 && bz == 4) {
#pragma unroll
    for (int z = 0; z < 4; z++)
#pragma unroll
      for (int y = 0; y < 4; y++) {
        float4 v = make_float4(f[16 * z + 4 * y], f[16 * z + 4 * y + 1], f[16 * z + 4 * y + 2],
                               f[16 * z + 4 * y + 3]);
        *reinterpret_cast<float4*>(p + y * fd.sy + z * fd.sz) = v;
      }
  } else {
#pragma unroll
    for (int z = 0; z < 4; z++)
#pragma unroll
      for (int y = 0; y < 4; y++)
#pragma unroll
        for (int x = 0; x < 4; x++)
          if ((uint32_t)x < bx && (uint32_t)y < by && (uint32_t)z < bz)
            p[x * fd.sx + y * fd.sy + z * fd.sz] = f[16 * z + 4 * y + x];
  }
}

// ------------------------------------------------------------- kernels
// grid.x = ceil(nblocks/64) workgroups of one wavefront; dynamic LDS =
// (maxbits + 1) 64-bit words.
__global__ __launch_bounds__(64) void zfp_encode3_f32_kernel(const float* __restrict__ in, Field3 fd,
                                                             unsigned maxbits,
                                                             uint64_t* __restrict__ stream)
{
  extern __shared__ uint64_t lds[];
  const unsigned lane = threadIdx.x;
  const uint32_t first = blockIdx.x * 64u;
  const uint32_t valid = min(64u, fd.nblocks - first);

  for (unsigned i = lane; i <= maxbits; i += 64) lds[i] = 0;
  __syncthreads();

  if (lane < valid) {
    float f[64];
    load_block(in, fd, first + lane, f);
    LdsSink sink{lds, lane * maxbits, (maxbits & 63u) == 0};
    encode_block(f, maxbits, sink);
  }
  __syncthreads();

  const unsigned nwords = (valid * maxbits + 63u) >> 6;
  uint64_t* dst = stream + (size_t)blockIdx.x * maxbits;
  for (unsigned i = lane; i < nwords; i += 64) dst[i] = lds[i];
}

__global__ __launch_bounds__(64) void zfp_decode3_f32_kernel(const uint64_t* __restrict__ stream, Field3 fd,
                                                             unsigned maxbits, float* __restrict__ out)
{
  extern __shared__ uint64_t lds[];
  const unsigned lane = threadIdx.x;
  const uint32_t first = blockIdx.x * 64u;
  const uint32_t valid = min(64u, fd.nblocks - first);

  const unsigned nwords = (valid * maxbits + 63u) >> 6;
  const uint64_t* src = stream + (size_t)blockIdx.x * maxbits;
  for (unsigned i = lane; i <= maxbits; i += 64) lds[i] = i < nwords ? src[i] : 0;
  __syncthreads();

  if (lane < valid) {
    float f[64];
    LdsSource source{lds, lane * maxbits};
    decode_block(source, maxbits, f);
    store_block(out, fd, first + lane, f);
  }
}

// ------------------------------------------------------------- host side
static int make_field(Field3& fd, const void* base, size_t nx, size_t ny, size_t nz, ptrdiff_t sx,
                      ptrdiff_t sy, ptrdiff_t sz, unsigned maxbits)
{
  if (!nx || !ny || !nz) return CSWAP_E_ARG;
  if (maxbits < 16 || maxbits > 4096) return CSWAP_E_ARG;
  if (nx > 0x7fffffffu || ny > 0x7fffffffu || nz > 0x7fffffffu) return CSWAP_E_ARG;
  size_t mx = (nx + 3) / 4, my = (ny + 3) / 4, mz = (nz + 3) / 4;
  size_t nb = mx * my * mz;
  if (nb / mz != mx * my || nb > 0xfffffff0ull) return CSWAP_E_ARG;
  fd.nx = (uint32_t)nx; fd.ny = (uint32_t)ny; fd.nz = (uint32_t)nz;
  fd.mx = (uint32_t)mx; fd.my = (uint32_t)my;
  fd.nblocks = (uint32_t)nb;
  fd.sx = sx ? sx : 1;
  fd.sy = sy ? sy : (ptrdiff_t)nx;
  fd.sz = sz ? sz : (ptrdiff_t)(nx * ny);
  fd.rows16 = fd.sx == 1 && (fd.sy % 4) == 0 && (fd.sz % 4) == 0 && ((uintptr_t)base % 16) == 0;
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

extern "C" int cswap_zfp_compress_f32(const float* d_in, size_t nx, size_t ny, size_t nz, ptrdiff_t sx,
                                      ptrdiff_t sy, ptrdiff_t sz, unsigned maxbits, uint64_t* d_stream,
                                      cswap_stream_t stream)
{
  if (!d_in || !d_stream) return CSWAP_E_ARG;
  Field3 fd;
  int rc = make_field(fd, d_in, nx, ny, nz, sx, sy, sz, maxbits);
  if (rc) return rc;
  unsigned grid = (fd.nblocks + 63) / 64;
  size_t lds_bytes = ((size_t)maxbits + 1) * 8;
  hipLaunchKernelGGL(zfp_encode3_f32_kernel, dim3(grid), dim3(64), lds_bytes, (hipStream_t)stream, d_in, fd,
                     maxbits, d_stream);
  return check_launch();
}

extern "C" int cswap_zfp_decompress_f32(const uint64_t* d_stream, size_t nx, size_t ny, size_t nz,
                                        ptrdiff_t sx, ptrdiff_t sy, ptrdiff_t sz, unsigned maxbits,
                                        float* d_out, cswap_stream_t stream)
{
  if (!d_out || !d_stream) return CSWAP_E_ARG;
  Field3 fd;
  int rc = make_field(fd, d_out, nx, ny, nz, sx, sy, sz, maxbits);
  if (rc) return rc;
  unsigned grid = (fd.nblocks + 63) / 64;
  size_t lds_bytes = ((size_t)maxbits + 1) * 8;
  hipLaunchKernelGGL(zfp_decode3_f32_kernel, dim3(grid), dim3(64), lds_bytes, (hipStream_t)stream, d_stream,
                     fd, maxbits, d_out);
  return check_launch();
}
