// compat.cpp -- the reference's entry-point names as adapters over the C ABI.
#include <atomic>
#include "common.h"
#define CSWAP_COMPAT_NO_PROTOTYPES
#include "../../include/cswap_compat.h"

namespace {
void* default_alloc(size_t b)
{
  void* p = nullptr;
  return hipMalloc(&p, b) == hipSuccess ? p : nullptr;
}
void default_free(void* p) { (void)hipFree(p); }

std::atomic<void* (*)(size_t)> g_alloc{default_alloc};
std::atomic<void (*)(void*)> g_free{default_free};
std::atomic<unsigned> g_maxbits{512};
std::atomic<size_t> g_nx{0}, g_ny{0};

bool is_device_ptr(const void* p)
{
  hipPointerAttribute_t a;
  if (hipPointerGetAttributes(&a, p) != hipSuccess) {
    (void)hipGetLastError();  // unregistered host memory reports an error: clear it
    return false;
  }
  return a.type == hipMemoryTypeDevice || a.type == hipMemoryTypeManaged;
}

// number of dimensions = leading non-zero extents, as zfp_field_dimensionality
// (zfp/zfp.c:60-64); 0 for an empty or 4-D field
int field_dims_of(const cswap_zfp_field* f)
{
  if (!f->nx || f->nw) return 0;
  if (!f->ny) return f->nz ? 0 : 1;
  return f->nz ? 3 : 2;
}

size_t field_elems(const cswap_zfp_field* f)
{
  return f->nx * (f->ny ? f->ny : 1) * (f->nz ? f->nz : 1);
}

bool host_field_contiguous(const cswap_zfp_field* f)
{
  return !((f->sx && f->sx != 1) || (f->ny && f->sy && f->sy != (ptrdiff_t)f->nx) ||
           (f->nz && f->sz && f->sz != (ptrdiff_t)(f->nx * f->ny)));
}

void flat_dims(long long numel, size_t& nx, size_t& ny, size_t& nz)
{
  size_t n = (size_t)numel;
  size_t ux = g_nx.load(), uy = g_ny.load();
  if (ux && uy && n % (ux * uy) == 0) { nx = ux; ny = uy; nz = n / (ux * uy); return; }
  if (n % 1024 == 0) { nx = 32; ny = 32; nz = n / 1024; return; }
  if (n % 16 == 0) { nx = 4; ny = 4; nz = n / 16; return; }
  nx = n; ny = 1; nz = 1;
}
}  // namespace

extern "C" {

void cswap_set_allocator(void* (*alloc_fn)(size_t), void (*free_fn)(void*))
{
  g_alloc.store(alloc_fn ? alloc_fn : default_alloc);
  g_free.store(free_fn ? free_fn : default_free);
}

void cswap_compat_set_field(size_t nx, size_t ny)
{
  g_nx.store(nx);
  g_ny.store(ny);
}

void PreGPUcompression(int arraySize, int kernelSize, float* arrayGPU, int* valueIndex, int, int, void* stream)
{
  (void)cswap_zvc_count(arrayGPU, arraySize, kernelSize, valueIndex, stream);
}

void PreAcc(int* valueIndex, int KernelSize, int* num, int, int, void* stream)
{
  (void)cswap_zvc_scan(valueIndex, KernelSize, num, stream);
}

void GPUcompression(int arraySize, int kernelSize, float* arrayGPU, float* compressedList,
                    int* compressedValueIndex, uint32_t* compressedBinIndex, int, int, void* stream)
{
  (void)cswap_zvc_compact(arrayGPU, arraySize, kernelSize, compressedValueIndex, compressedList,
                          compressedBinIndex, stream);
}

void GPUdecompression(float* arrayGPU, float* destiGPU, int arraySize, int kernelSize, uint32_t* gpuDataindex,
                      int* beginIndex, int, int)
{
  (void)cswap_zvc_expand(arrayGPU, gpuDataindex, beginIndex, arraySize, kernelSize, destiGPU, nullptr);
}

void setRatio(int ratio)
{
  if (ratio > 0 && 4 * ratio >= 16 && 4 * ratio <= 4096) g_maxbits.store((unsigned)(4 * ratio));
}

size_t cuda_compress(cswap_zfp_stream* zs, const cswap_zfp_field* f)
{
  if (!zs || !f || !zs->stream || !f->data || !zs->stream->begin) return 0;
  const int dims = field_dims_of(f);
  // fields of 1, 2 or 3 dimensions of any of the four scalar types the reference
  // dispatches on (cuZFP.cu:389-423): zfp_type_int32 = 1, int64 = 2, float = 3, double = 4
  if (f->type < 1 || f->type > 4 || !dims) return 0;
  const size_t esz = (f->type == 1 || f->type == 3) ? 4 : 8;
  const unsigned maxbits = zs->maxbits;
  const size_t cap = cswap_zfp_stream_capacity_nd(dims, f->nx, f->ny, f->nz, maxbits);
  const size_t bytes = cswap_zfp_stream_bytes_nd(dims, f->nx, f->ny, f->nz, maxbits);
  const bool field_dev = is_device_ptr(f->data), stream_dev = is_device_ptr(zs->stream->begin);
  const void* d_in = f->data;
  uint64_t* d_stream = zs->stream->begin;
  void *tmp_in = nullptr, *tmp_s = nullptr;
  size_t ok = 0;
  do {
    if (!field_dev) {  // host field: contiguous only, staged like zfp/cuZFP.cu:265-312
      if (!host_field_contiguous(f)) break;
      size_t fb = esz * field_elems(f);
      if (hipMalloc(&tmp_in, fb) != hipSuccess) break;
      if (hipMemcpy(tmp_in, f->data, fb, hipMemcpyHostToDevice) != hipSuccess) break;
      d_in = tmp_in;
    }
    if (!stream_dev) {
      if (hipMalloc(&tmp_s, cap) != hipSuccess) break;
      d_stream = (uint64_t*)tmp_s;
    }
    const ptrdiff_t sx = field_dev ? f->sx : 0, sy = field_dev ? f->sy : 0, sz = field_dev ? f->sz : 0;
    int rc;
    switch (f->type) {
      case 1: rc = cswap_zfp_compress_i32_nd((const int32_t*)d_in, dims, f->nx, f->ny, f->nz, sx, sy, sz, maxbits, d_stream, nullptr); break;
      case 2: rc = cswap_zfp_compress_i64_nd((const int64_t*)d_in, dims, f->nx, f->ny, f->nz, sx, sy, sz, maxbits, d_stream, nullptr); break;
      case 3: rc = cswap_zfp_compress_f32_nd((const float*)d_in, dims, f->nx, f->ny, f->nz, sx, sy, sz, maxbits, d_stream, nullptr); break;
      default: rc = cswap_zfp_compress_f64_nd((const double*)d_in, dims, f->nx, f->ny, f->nz, sx, sy, sz, maxbits, d_stream, nullptr); break;
    }
    if (rc) break;
    if (!stream_dev) {
      if (hipMemcpy(zs->stream->begin, tmp_s, cap, hipMemcpyDeviceToHost) != hipSuccess) break;
    } else if (hipStreamSynchronize(nullptr) != hipSuccess) {
      break;
    }
    ok = bytes;
  } while (0);
  if (tmp_in) (void)hipFree(tmp_in);
  if (tmp_s) (void)hipFree(tmp_s);
  if (ok) {  // zfp/cuZFP.cu:428-433
    zs->stream->bits = 64;
    zs->stream->ptr = zs->stream->begin + ok / 8;
  }
  return ok;
}

void cuda_decompress(cswap_zfp_stream* zs, cswap_zfp_field* f)
{
  if (!zs || !f || !zs->stream || !f->data || !zs->stream->begin) return;
  const int dims = field_dims_of(f);
  if (f->type < 1 || f->type > 4 || !dims) return;
  const size_t esz = (f->type == 1 || f->type == 3) ? 4 : 8;
  const unsigned maxbits = zs->maxbits;
  const size_t cap = cswap_zfp_stream_capacity_nd(dims, f->nx, f->ny, f->nz, maxbits);
  const size_t bytes = cswap_zfp_stream_bytes_nd(dims, f->nx, f->ny, f->nz, maxbits);
  const bool field_dev = is_device_ptr(f->data), stream_dev = is_device_ptr(zs->stream->begin);
  void* d_out = f->data;
  const uint64_t* d_stream = zs->stream->begin;
  void *tmp_out = nullptr, *tmp_s = nullptr;
  const size_t fb = esz * field_elems(f);
  bool ok = false;
  do {
    if (!field_dev) {
      if (!host_field_contiguous(f)) break;
      if (hipMalloc(&tmp_out, fb) != hipSuccess) break;
      d_out = tmp_out;
    }
    if (!stream_dev) {
      if (hipMalloc(&tmp_s, cap) != hipSuccess) break;
      if (hipMemcpy(tmp_s, zs->stream->begin, cap, hipMemcpyHostToDevice) != hipSuccess) break;
      d_stream = (const uint64_t*)tmp_s;
    }
    const ptrdiff_t sx = field_dev ? f->sx : 0, sy = field_dev ? f->sy : 0, sz = field_dev ? f->sz : 0;
    int rc;
    switch (f->type) {
      case 1: rc = cswap_zfp_decompress_i32_nd(d_stream, dims, f->nx, f->ny, f->nz, sx, sy, sz, maxbits, (int32_t*)d_out, nullptr); break;
      case 2: rc = cswap_zfp_decompress_i64_nd(d_stream, dims, f->nx, f->ny, f->nz, sx, sy, sz, maxbits, (int64_t*)d_out, nullptr); break;
      case 3: rc = cswap_zfp_decompress_f32_nd(d_stream, dims, f->nx, f->ny, f->nz, sx, sy, sz, maxbits, (float*)d_out, nullptr); break;
      default: rc = cswap_zfp_decompress_f64_nd(d_stream, dims, f->nx, f->ny, f->nz, sx, sy, sz, maxbits, (double*)d_out, nullptr); break;
    }
    if (rc) break;
    if (!field_dev) {
      if (hipMemcpy(f->data, tmp_out, fb, hipMemcpyDeviceToHost) != hipSuccess) break;
    } else if (hipStreamSynchronize(nullptr) != hipSuccess) {
      break;
    }
    ok = true;
  } while (0);
  if (tmp_out) (void)hipFree(tmp_out);
  if (tmp_s) (void)hipFree(tmp_s);
  if (ok) {  // zfp/cuZFP.cu:527-531: success is signalled by advancing the stream pointer
    zs->stream->bits = 64;
    zs->stream->ptr = zs->stream->begin + bytes / 8;
  }
}

void* compress(void* dev_ptr, long long numel, size_t* out_bytes)
{
  if (!dev_ptr || numel <= 0 || !out_bytes) return nullptr;
  size_t nx, ny, nz;
  flat_dims(numel, nx, ny, nz);
  const unsigned maxbits = g_maxbits.load();
  const size_t cap = cswap_zfp_stream_capacity(nx, ny, nz, maxbits);
  void* buf = g_alloc.load()(cap);
  if (!buf) return nullptr;
  if (cswap_zfp_compress_f32((const float*)dev_ptr, nx, ny, nz, 0, 0, 0, maxbits, (uint64_t*)buf, nullptr) ||
      hipStreamSynchronize(nullptr) != hipSuccess) {
    g_free.load()(buf);
    return nullptr;
  }
  *out_bytes = cap;
  return buf;
}

int decompress(const void* dev_buffer, long long numel, void* dev_out)
{
  if (!dev_buffer || numel <= 0 || !dev_out) return CSWAP_E_ARG;
  size_t nx, ny, nz;
  flat_dims(numel, nx, ny, nz);
  int rc = cswap_zfp_decompress_f32((const uint64_t*)dev_buffer, nx, ny, nz, 0, 0, 0, g_maxbits.load(),
                                    (float*)dev_out, nullptr);
  if (rc) return rc;
  return hipStreamSynchronize(nullptr) == hipSuccess ? CSWAP_OK : CSWAP_E_HIP;
}

}  // extern "C"
