// zvc_kernels.hip -- zero-value compaction (ZVC) of fp32 tensors for gfx950, in
// the reference's on-the-wire format (CSWAP+/zfp/compression.cu): the tensor is
// cut into `process` contiguous chunks of E = ceil(n/process) elements; chunk i
// owns W = ceil(E/32) mask words at word i*W (bit k%32 of word k/32 <=> element
// E*i+k != 0) and its packed non-zeros start at values[begin[i]].
//
// Work decomposition: ONE WAVEFRONT PER CHUNK (the reference uses one thread
// per chunk, which makes every access strided by E).  Lane l of iteration t
// looks at chunk element 64t+l, so loads are contiguous 256-byte rows, one
// __ballot gives the two mask words of the iteration directly in the
// reference's bit order, mbcnt gives each non-zero its slot, and the packed
// stores of a wave are contiguous.  The chunk-granular exclusive scan the
// format carries anyway (`begin`) is the device-wide scan; no finer scan is
// needed.
#include <hip/hip_runtime.h>
#include "../../include/cswap_hip.h"
#include "common.h"

namespace cswap {

constexpr int kWavesPerGroup = 4;

__device__ __forceinline__ unsigned lane_id() { return threadIdx.x & 63u; }
__device__ __forceinline__ unsigned popc64(unsigned long long v) { return (unsigned)__popcll(v); }
// number of set bits of m below this lane
__device__ __forceinline__ unsigned rank_below(unsigned long long m)
{
  return __builtin_amdgcn_mbcnt_hi((unsigned)(m >> 32), __builtin_amdgcn_mbcnt_lo((unsigned)m, 0u));
}

__device__ __forceinline__ int wave_sum(int v)
{
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

struct Geometry {
  int n;        // elements
  int E;        // elements per chunk
  int W;        // mask words per chunk
  int process;  // chunks in the layout
  int active;   // chunks that hold data
};

// ------------------------------------------------------------------ count
__global__ __launch_bounds__(64 * kWavesPerGroup) void zvc_count_kernel(const float* __restrict__ in,
                                                                         Geometry g, int* __restrict__ count)
{
  const int c = blockIdx.x * kWavesPerGroup + (threadIdx.x >> 6);
  if (c >= g.active) return;
  const unsigned lane = lane_id();
  const long long b = (long long)g.E * c;
  const int len = (int)min((long long)g.E, (long long)g.n - b);
  const float* p = in + b;
  int acc = 0;
  if ((((uintptr_t)p) & 15u) == 0) {
    const float4* p4 = reinterpret_cast<const float4*>(p);
    const int n4 = len >> 2;
    for (int i = lane; i < n4; i += 64) {
      float4 v = p4[i];
      acc += (v.x != 0.0f) + (v.y != 0.0f) + (v.z != 0.0f) + (v.w != 0.0f);
    }
    for (int i = (n4 << 2) + lane; i < len; i += 64) acc += (p[i] != 0.0f);
  } else {
    for (int i = lane; i < len; i += 64) acc += (p[i] != 0.0f);
  }
  acc = wave_sum(acc);
  if (lane == 0) count[c] = acc;
}

// ------------------------------------------------------------------ scan
// In-place exclusive scan of k ints by one workgroup; total to *nnz.
__global__ __launch_bounds__(1024) void zvc_scan_kernel(int* __restrict__ v, int k, int* __restrict__ nnz)
{
  __shared__ int wave_tot[16];
  __shared__ int carry_s;
  const unsigned tid = threadIdx.x, lane = tid & 63u, wv = tid >> 6;
  if (tid == 0) carry_s = 0;
  __syncthreads();
  for (int base = 0; base < k; base += 1024) {
    int i = base + (int)tid;
    int x = i < k ? v[i] : 0;
    // inclusive scan inside the wave
    int s = x;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      int t = __shfl_up(s, o, 64);
      if ((int)lane >= o) s += t;
    }
    if (lane == 63) wave_tot[wv] = s;
    __syncthreads();
    int wave_off = 0;
    for (unsigned w = 0; w < wv; w++) wave_off += wave_tot[w];
    int carry = carry_s;
    if (i < k) v[i] = carry + wave_off + s - x;
    __syncthreads();
    if (tid == 1023) carry_s = carry + wave_off + s;
    __syncthreads();
  }
  if (tid == 0) *nnz = carry_s;
}

// ------------------------------------------------------------------ compact
__global__ __launch_bounds__(64 * kWavesPerGroup) void zvc_compact_kernel(
    const float* __restrict__ in, Geometry g, const int* __restrict__ begin, float* __restrict__ values,
    uint32_t* __restrict__ mask)
{
  const int c = blockIdx.x * kWavesPerGroup + (threadIdx.x >> 6);
  if (c >= g.process) return;
  const unsigned lane = lane_id();
  uint32_t* mrow = mask + (size_t)c * g.W;
  if (c >= g.active) {  // chunk without data: the reference leaves these words untouched; define them
    for (int w = lane; w < g.W; w += 64) mrow[w] = 0;
    return;
  }
  const long long b = (long long)g.E * c;
  const int len = (int)min((long long)g.E, (long long)g.n - b);
  const float* p = in + b;
  unsigned off = (unsigned)begin[c];
  const int iters = (g.E + 63) >> 6;
  uint32_t held = 0;  // lane l holds mask word (64*(t/32) + l) of the chunk until flushed
  for (int t = 0; t < iters; t++) {
    const int k = t * 64 + (int)lane;
    const bool valid = k < len;
    const float x = valid ? p[k] : 0.0f;
    const bool nz = valid && (x != 0.0f);
    const unsigned long long m = __ballot(nz);
    if (nz) values[off + rank_below(m)] = x;
    off += popc64(m);
    const unsigned slot = (unsigned)(2 * t) & 63u;
    if (lane == slot) held = (uint32_t)m;
    if (lane == slot + 1) held = (uint32_t)(m >> 32);
    if ((t & 31) == 31 || t == iters - 1) {
      const int w = (t >> 5) * 64 + (int)lane;
      const int filled = 2 * (t & 31) + 2;
      if ((int)lane < filled && w < g.W) mrow[w] = held;
      held = 0;
    }
  }
}

// ------------------------------------------------------------------ expand
__global__ __launch_bounds__(64 * kWavesPerGroup) void zvc_expand_kernel(
    const float* __restrict__ values, const uint32_t* __restrict__ mask, const int* __restrict__ begin,
    Geometry g, float* __restrict__ out)
{
  const int c = blockIdx.x * kWavesPerGroup + (threadIdx.x >> 6);
  if (c >= g.active) return;
  const unsigned lane = lane_id();
  const long long b = (long long)g.E * c;
  const int len = (int)min((long long)g.E, (long long)g.n - b);
  const uint32_t* mrow = mask + (size_t)c * g.W;
  float* q = out + b;
  unsigned off = (unsigned)begin[c];
  const int iters = (len + 63) >> 6;
  uint32_t held = 0;
  for (int t = 0; t < iters; t++) {
    if ((t & 31) == 0) {  // refill: lane l takes mask word 64*(t/32)+l of this chunk
      const int w = (t >> 5) * 64 + (int)lane;
      held = w < g.W ? mrow[w] : 0u;
    }
    const unsigned slot = (unsigned)(2 * t) & 63u;
    const uint32_t lo = (uint32_t)__shfl((int)held, (int)slot, 64);
    const uint32_t hi = (uint32_t)__shfl((int)held, (int)slot + 1, 64);
    const int k = t * 64 + (int)lane;
    // bits past the end of the chunk carry no data
    const int rem = len - t * 64;
    unsigned long long m = ((unsigned long long)hi << 32) | lo;
    if (rem < 64) m &= (1ull << rem) - 1ull;
    const bool nz = (m >> lane) & 1ull;
    const float x = nz ? values[off + rank_below(m)] : 0.0f;
    if (k < len) q[k] = x;
    off += popc64(m);
  }
}

// ------------------------------------------------------------------ probe
__global__ void zero_u64_kernel(unsigned long long* p) { *p = 0ull; }

__global__ __launch_bounds__(256) void probe_nnz_kernel(const float* __restrict__ in, size_t n,
                                                        unsigned long long* __restrict__ nnz)
{
  const size_t tid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t nthreads = (size_t)gridDim.x * blockDim.x;
  unsigned acc = 0;
  // head up to 16-byte alignment, body in float4, tail
  size_t head = (16 - ((uintptr_t)in & 15u)) & 15u;
  head = min(head >> 2, n);
  for (size_t i = tid; i < head; i += nthreads) acc += (in[i] != 0.0f);
  const float4* p4 = reinterpret_cast<const float4*>(in + head);
  const size_t n4 = (n - head) >> 2;
  for (size_t i = tid; i < n4; i += nthreads) {
    float4 v = p4[i];
    acc += (v.x != 0.0f) + (v.y != 0.0f) + (v.z != 0.0f) + (v.w != 0.0f);
  }
  for (size_t i = head + (n4 << 2) + tid; i < n; i += nthreads) acc += (in[i] != 0.0f);
  acc = (unsigned)wave_sum((int)acc);
  __shared__ unsigned part[4];
  if ((threadIdx.x & 63u) == 0) part[threadIdx.x >> 6] = acc;
  __syncthreads();
  if (threadIdx.x == 0) {
    unsigned long long s = (unsigned long long)part[0] + part[1] + part[2] + part[3];
    if (s) atomicAdd(nnz, s);
  }
}

static int make_geometry(Geometry& g, int n, int process)
{
  if (n <= 0 || process <= 0 || process > (1 << 20)) return CSWAP_E_ARG;
  g.n = n;
  g.process = process;
  g.E = n / process + (n % process != 0);
  g.W = g.E / 32 + (g.E % 32 != 0);
  g.active = n / g.E + (n % g.E != 0);
  return CSWAP_OK;
}

}  // namespace cswap

using namespace cswap;

extern "C" int cswap_zvc_chunk_elems(int n, int process)
{
  Geometry g;
  return make_geometry(g, n, process) ? 0 : g.E;
}
extern "C" int cswap_zvc_chunk_words(int n, int process)
{
  Geometry g;
  return make_geometry(g, n, process) ? 0 : g.W;
}
extern "C" int cswap_zvc_active_chunks(int n, int process)
{
  Geometry g;
  return make_geometry(g, n, process) ? 0 : g.active;
}
extern "C" size_t cswap_zvc_mask_bytes(int n, int process)
{
  Geometry g;
  return make_geometry(g, n, process) ? 0 : (size_t)g.W * (size_t)g.process * sizeof(uint32_t);
}

extern "C" int cswap_zvc_count(const float* d_in, int n, int process, int* d_count, cswap_stream_t stream)
{
  if (!d_in || !d_count) return CSWAP_E_ARG;
  Geometry g;
  int rc = make_geometry(g, n, process);
  if (rc) return rc;
  unsigned grid = (g.active + kWavesPerGroup - 1) / kWavesPerGroup;
  hipLaunchKernelGGL(zvc_count_kernel, dim3(grid), dim3(64 * kWavesPerGroup), 0, (hipStream_t)stream, d_in, g,
                     d_count);
  return check_launch();
}

extern "C" int cswap_zvc_scan(int* d_count, int k, int* d_nnz, cswap_stream_t stream)
{
  if (!d_count || !d_nnz || k <= 0) return CSWAP_E_ARG;
  hipLaunchKernelGGL(zvc_scan_kernel, dim3(1), dim3(1024), 0, (hipStream_t)stream, d_count, k, d_nnz);
  return check_launch();
}

extern "C" int cswap_zvc_compact(const float* d_in, int n, int process, const int* d_begin, float* d_values,
                                 uint32_t* d_mask, cswap_stream_t stream)
{
  if (!d_in || !d_begin || !d_values || !d_mask) return CSWAP_E_ARG;
  Geometry g;
  int rc = make_geometry(g, n, process);
  if (rc) return rc;
  unsigned grid = (g.process + kWavesPerGroup - 1) / kWavesPerGroup;
  hipLaunchKernelGGL(zvc_compact_kernel, dim3(grid), dim3(64 * kWavesPerGroup), 0, (hipStream_t)stream, d_in,
                     g, d_begin, d_values, d_mask);
  return check_launch();
}

extern "C" int cswap_zvc_expand(const float* d_values, const uint32_t* d_mask, const int* d_begin, int n,
                                int process, float* d_out, cswap_stream_t stream)
{
  if (!d_values || !d_mask || !d_begin || !d_out) return CSWAP_E_ARG;
  Geometry g;
  int rc = make_geometry(g, n, process);
  if (rc) return rc;
  unsigned grid = (g.active + kWavesPerGroup - 1) / kWavesPerGroup;
  hipLaunchKernelGGL(zvc_expand_kernel, dim3(grid), dim3(64 * kWavesPerGroup), 0, (hipStream_t)stream,
                     d_values, d_mask, d_begin, g, d_out);
  return check_launch();
}

extern "C" int cswap_zvc_compress(const float* d_in, int n, int process, int* d_begin, int* d_nnz,
                                  float* d_values, uint32_t* d_mask, cswap_stream_t stream)
{
  if (!d_nnz) return CSWAP_E_ARG;
  int rc = cswap_zvc_count(d_in, n, process, d_begin, stream);
  if (rc) return rc;
  rc = cswap_zvc_scan(d_begin, cswap_zvc_active_chunks(n, process), d_nnz, stream);
  if (rc) return rc;
  return cswap_zvc_compact(d_in, n, process, d_begin, d_values, d_mask, stream);
}

extern "C" int cswap_probe_nnz(const float* d_in, size_t n, unsigned long long* d_nnz, cswap_stream_t stream)
{
  if (!d_in || !d_nnz || !n) return CSWAP_E_ARG;
  hipLaunchKernelGGL(zero_u64_kernel, dim3(1), dim3(1), 0, (hipStream_t)stream, d_nnz);
  size_t want = (n / 4 + 255) / 256;
  unsigned grid = (unsigned)(want < 1 ? 1 : (want > 256 * 16 ? 256 * 16 : want));
  hipLaunchKernelGGL(probe_nnz_kernel, dim3(grid), dim3(256), 0, (hipStream_t)stream, d_in, n, d_nnz);
  return check_launch();
}
