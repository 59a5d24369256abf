/*
 * cswap_compat.h -- the reference's own entry-point names, exported by
 * libcswap_hip.so so that the call sites of the patched training loop
 * (CSWAP+/Execution.h:23-27,63,88-95,113 and CSWAP+/simple.c:63,74) link
 * against the HIP implementation unchanged, with hipStream_t where the
 * reference takes cudaStream_t.  They are thin adapters over cswap_hip.h.
 *
 * The struct types below have the memory layout of the reference's zfp_stream,
 * zfp_field and bitstream (CSWAP+/zfp/zfp.h:79-145, CSWAP+/zfp/bitstream.c:135-146)
 * under other names, so this header can be included next to the reference's
 * zfp.h; code that already includes zfp.h passes its own zfp_stream* / zfp_field*.
 */
#ifndef CSWAP_COMPAT_H
#define CSWAP_COMPAT_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct {
  unsigned bits;      /* buffered bits */
  uint64_t buffer;
  uint64_t* ptr;      /* next word */
  uint64_t* begin;    /* start of the stream: DEVICE or host memory */
  uint64_t* end;
} cswap_bitstream;

typedef struct {
  unsigned minbits, maxbits, maxprec;
  int minexp;
  cswap_bitstream* stream;
  struct { int policy; struct { unsigned threads, chunk_size; } omp; } exec;
} cswap_zfp_stream;

typedef struct {
  int type;                 /* zfp_type: 1 = int32, 2 = int64, 3 = float, 4 = double (cuZFP.cu:389-423) */
  size_t nx, ny, nz, nw;
  ptrdiff_t sx, sy, sz, sw; /* 0 = contiguous */
  void* data;               /* DEVICE or host memory */
} cswap_zfp_field;

#ifndef CSWAP_COMPAT_NO_PROTOTYPES
/* CSWAP+/zfp/compression.cuh:4-9.  kernelSize is the number of chunks
 * (the reference passes dimsize*blocksize = 16384); dimsize/blocksize are the
 * reference's launch geometry and are ignored (one wavefront works per chunk). */
void PreGPUcompression(int arraySize, int kernelSize, float* arrayGPU, int* valueIndex, int dimsize,
                       int blocksize, void* stream);
void PreAcc(int* valueIndex, int KernelSize, int* num, int dimsize, int blocksize, void* stream);
void GPUcompression(int arraySize, int kernelSize, float* arrayGPU, float* compressedList,
                    int* compressedValueIndex, uint32_t* compressedBinIndex, int dimsize, int blocksize,
                    void* stream);
/* runs on the default stream like the reference (compression.cu:372); unlike
 * it, writes every output element */
void GPUdecompression(float* arrayGPU, float* destiGPU, int arraySize, int kernelSize, uint32_t* gpuDataindex,
                      int* beginIndex, int dimsize, int blocksize);

/* CSWAP+/zfp/cuZFP.h:11-12.  Float fields of 1, 2 or 3 dimensions (trailing zero
 * extents, zfp/zfp.c:60-64); returns the stream size in bytes
 * (0 = failure) and, like the reference, has finished when it returns. */
size_t cuda_compress(cswap_zfp_stream* stream, const cswap_zfp_field* field);
void   cuda_decompress(cswap_zfp_stream* stream, cswap_zfp_field* field);

/* libtorch-facing wrappers whose definitions are absent from the reference tree
 * (ATen/core/zfp.h; call sites CSWAP+/Execution.h:63,113,201). */
void  setRatio(int ratio);                 /* bits per 4x4x4 block = 4*ratio: 128 -> 8 bits/value */
void* compress(void* dev_ptr, long long numel, size_t* out_bytes); /* returns a device buffer from the
                                              registered allocator; the caller frees it */
int   decompress(const void* dev_buffer, long long numel, void* dev_out);
#endif

/* Allocator `compress` draws its output buffer from (default hipMalloc/hipFree);
 * the patched loop registers torch's caching allocator raw_allocate/raw_deallocate
 * (CSWAP+/Execution.h:53-54,296). */
void cswap_set_allocator(void* (*alloc_fn)(size_t), void (*free_fn)(void*));
/* Field shape `compress`/`decompress` view a flat tensor as: nx, ny given, nz =
 * numel/(nx*ny).  0,0 restores the default (32x32 rows when numel is a multiple
 * of 1024, else 4x4, else numel x 1 x 1). */
void cswap_compat_set_field(size_t nx, size_t ny);

#ifdef __cplusplus
}
#endif

#if defined(__cplusplus) && !defined(CSWAP_COMPAT_NO_PROTOTYPES)
/* The form the reference's call sites use,
 *   buffer = compress(pre.data_ptr(), pre.numel(), buffersize);
 * (CSWAP+/Execution.h:113,201: the size comes back through a size_t lvalue), so
 * that those lines compile unchanged. */
inline void* compress(void* dev_ptr, long long numel, size_t& out_bytes)
{
  return compress(dev_ptr, numel, &out_bytes);
}
#endif
#endif /* CSWAP_COMPAT_H */
