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
#include <atomic>

#include <mutex>

#include "../../include/cswap_hip.h"
#include "../../include/cswap_test_hooks.h"
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

// 16-byte store with the nontemporal hint, for output that is written once in whole lines
typedef float stream_f4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void st_stream4(float4* p, float4 v)
{
  stream_f4 t = {v.x, v.y, v.z, v.w};
  __builtin_nontemporal_store(t, reinterpret_cast<stream_f4*>(p));
}

struct Geometry {
  int n;        // elements
  int E;        // elements per chunk
  int W;        // mask words per chunk
  int process;  // chunks in the layout
  int active;   // chunks that hold data
  int backwards;  // compaction order, see zvc_compact_kernel
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
// In-place exclusive scan of k ints by one workgroup of 1024 threads; total to
// *nnz.  Each thread owns 16 consecutive entries per 16384-entry tile.
__global__ __launch_bounds__(1024) void zvc_scan_kernel(int* __restrict__ v, int k, int* __restrict__ nnz)
{
  __shared__ int wave_tot[16];
  const unsigned tid = threadIdx.x, lane = tid & 63u, wv = tid >> 6;
  int carry = 0;
  for (int base = 0; base < k; base += 16384) {
    const int i0 = base + (int)tid * 16;
    int x[16];
    if (i0 + 16 <= k) {
      const int4* p = reinterpret_cast<const int4*>(v + i0);
#pragma unroll
      for (int j = 0; j < 4; j++) {
        int4 q = p[j];
        x[4 * j] = q.x; x[4 * j + 1] = q.y; x[4 * j + 2] = q.z; x[4 * j + 3] = q.w;
      }
    } else {
#pragma unroll
      for (int j = 0; j < 16; j++) x[j] = i0 + j < k ? v[i0 + j] : 0;
    }
    int tsum = 0;
#pragma unroll
    for (int j = 0; j < 16; j++) tsum += x[j];
    int s = tsum;  // inclusive scan of thread sums inside the wave
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      int t = __shfl_up(s, o, 64);
      if ((int)lane >= o) s += t;
    }
    __syncthreads();  // wave_tot of the previous tile has been consumed
    if (lane == 63) wave_tot[wv] = s;
    __syncthreads();
    int wave_off = 0, total = 0;
#pragma unroll
    for (unsigned w = 0; w < 16; w++) {
      int t = wave_tot[w];
      if (w < wv) wave_off += t;
      total += t;
    }
    int run = carry + wave_off + s - tsum;
    if (i0 + 16 <= k) {
      int4* p = reinterpret_cast<int4*>(v + i0);
#pragma unroll
      for (int j = 0; j < 4; j++) {
        int4 q;
        q.x = run; run += x[4 * j];
        q.y = run; run += x[4 * j + 1];
        q.z = run; run += x[4 * j + 2];
        q.w = run; run += x[4 * j + 3];
        p[j] = q;
      }
    } else {
#pragma unroll
      for (int j = 0; j < 16; j++) {
        if (i0 + j < k) v[i0 + j] = run;
        run += x[j];
      }
    }
    carry += total;
  }
  if (tid == 0) *nnz = carry;
}

// ------------------------------------------------------------------ compact
// Two forms.  zvc_compact_kernel (the one that normally runs) collects a chunk's
// non-zeros in a per-wave LDS ring of two 256-float halves and writes a half out
// whenever it is full: every lane stores 16 bytes of one aligned 1 KB run, with the
// nontemporal hint -- whole lines per store instruction, like the expansion's
// output.  The first and the last 16-byte group of a chunk may be shared with the
// neighbouring chunks and are written element by element.  It needs a 16-byte
// aligned values pointer; zvc_compact_rows_kernel below stores each row's non-zeros
// straight from the lanes that hold them and runs otherwise.
constexpr int kUnroll = 8;  // independent 256-byte rows in flight per wave
constexpr int kHalf = 256;  // floats per half of a wave's ring
// Tensors of at least this many bytes take the staged form.  Compaction alone / count + scan +
// compact, staged against row-wise, in microseconds: 512 MiB 177 / 240 against 166 / 254,
// 256 MiB 72 / 115 against 83 / 121, 128 MiB 33.6 / 57.9 against 32.1 / 56.5, 64 MiB 17.9 / 33.6
// against 17.0 / 32.7 (below the size of the memory-side cache the hint only costs: the
// next reader of the values finds them in HBM instead of the cache).
#ifndef CSWAP_STAGED_COMPACT_BYTES
#define CSWAP_STAGED_COMPACT_BYTES (192ull << 20)
#endif
static std::atomic<unsigned long long> g_staged_compact_bytes{CSWAP_STAGED_COMPACT_BYTES};  // cswap_zvc_set_staged_compact_bytes

__device__ __forceinline__ void lds_order()
{
  __builtin_amdgcn_wave_barrier();
  asm volatile("" ::: "memory");
}

__global__ __launch_bounds__(64 * kWavesPerGroup) void zvc_compact_kernel(
    const float* __restrict__ in, Geometry g, const int* __restrict__ begin, float* __restrict__ values,
    uint32_t* __restrict__ mask)
{
  __shared__ __attribute__((aligned(16))) float ring_all[kWavesPerGroup][2 * kHalf];
  int c = (int)(blockIdx.x * kWavesPerGroup + (threadIdx.x >> 6));
  if (c >= g.process) return;
  if (g.backwards) c = g.process - 1 - c;  // see zvc_compact_rows_kernel
  const unsigned lane = lane_id();
  float* ring = ring_all[threadIdx.x >> 6];
  uint32_t* mrow = mask + (size_t)c * g.W;
  if (c >= g.active) {
    for (int w = lane; w < g.W; w += 64) mrow[w] = 0;
    return;
  }
  const long long b = (long long)g.E * c;
  const int len = (int)min((long long)g.E, (long long)g.n - b);
  const float* p = in + b;
  const unsigned out0 = (unsigned)begin[c];
  unsigned skip = out0 & 3u;     // slots at the front of the next write-out that belong to the chunk before
  unsigned base = out0 - skip;   // index in values of the slot at `head` (a multiple of four)
  unsigned head = 0;             // 0 or kHalf
  unsigned fill = skip;          // slots in use, counted from head
  const int iters = (g.E + 63) >> 6;
  uint32_t held = 0;  // lane l holds mask word (64*(t/32) + l) of the chunk until flushed
  for (int t0 = 0; t0 < iters; t0 += kUnroll) {
    float x[kUnroll];
#pragma unroll
    for (int j = 0; j < kUnroll; j++) {
      const int k = (t0 + j) * 64 + (int)lane;
      x[j] = k < len ? p[k] : 0.0f;  // out-of-range elements read as zero: no bit, no value
    }
#pragma unroll
    for (int j = 0; j < kUnroll; j++) {
      const int t = t0 + j;
      const bool nz = x[j] != 0.0f;
      const unsigned long long m = __ballot(nz);
      if (nz) ring[(head + fill + rank_below(m)) & (2 * kHalf - 1)] = x[j];
      fill += popc64(m);
      if (fill >= (unsigned)kHalf) {  // wave-uniform: the half at head is complete
        lds_order();
        const stream_f4 v = *reinterpret_cast<const stream_f4*>(ring + head + 4 * lane);
        float* dst = values + base + 4 * lane;
        if (skip == 0) {
          __builtin_nontemporal_store(v, reinterpret_cast<stream_f4*>(dst));
        } else {
          const unsigned j0 = 4 * lane;
          if (j0 + 0 >= skip) dst[0] = v.x;
          if (j0 + 1 >= skip) dst[1] = v.y;
          if (j0 + 2 >= skip) dst[2] = v.z;
          if (j0 + 3 >= skip) dst[3] = v.w;
          skip = 0;
        }
        lds_order();
        base += kHalf;
        head ^= (unsigned)kHalf;
        fill -= (unsigned)kHalf;
      }
      if (t >= iters) continue;  // tail of the unrolled group: nothing left in this chunk
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
  // what is left in the ring: slots [skip, fill) of the half at head
  lds_order();
  const unsigned j0 = 4 * lane;
  if (j0 < fill) {
    const stream_f4 v = *reinterpret_cast<const stream_f4*>(ring + head + j0);
    float* dst = values + base + j0;
    if (j0 >= skip && j0 + 4 <= fill) {
      *reinterpret_cast<stream_f4*>(dst) = v;
    } else {
      if (j0 + 0 >= skip && j0 + 0 < fill) dst[0] = v.x;
      if (j0 + 1 >= skip && j0 + 1 < fill) dst[1] = v.y;
      if (j0 + 2 >= skip && j0 + 2 < fill) dst[2] = v.z;
      if (j0 + 3 >= skip && j0 + 3 < fill) dst[3] = v.w;
    }
  }
}


__global__ __launch_bounds__(64 * kWavesPerGroup) void zvc_compact_rows_kernel(
    const float* __restrict__ in, Geometry g, const int* __restrict__ begin, float* __restrict__ values,
    uint32_t* __restrict__ mask)
{
  // Tensors larger than the memory-side cache are walked from the last chunk
  // to the first: the counting pass that ran just before went first to last, so
  // the chunks it touched last are the ones still cached (measured: count + scan
  // + compact 6-7 % faster at 256 and 512 MiB; smaller tensors stay cached
  // either way and are walked forwards).
  int c = (int)(blockIdx.x * kWavesPerGroup + (threadIdx.x >> 6));
  if (c >= g.process) return;
  if (g.backwards) c = g.process - 1 - c;
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
  for (int t0 = 0; t0 < iters; t0 += kUnroll) {
    float x[kUnroll];
#pragma unroll
    for (int j = 0; j < kUnroll; j++) {
      const int k = (t0 + j) * 64 + (int)lane;
      x[j] = k < len ? p[k] : 0.0f;  // out-of-range elements read as zero: no bit, no value
    }
#pragma unroll
    for (int j = 0; j < kUnroll; j++) {
      const int t = t0 + j;
      const bool nz = x[j] != 0.0f;
      const unsigned long long m = __ballot(nz);
      if (nz) values[off + rank_below(m)] = x[j];
      off += popc64(m);
      if (t >= iters) continue;  // tail of the unrolled group: nothing left in this chunk
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
  for (int t0 = 0; t0 < iters; t0 += kUnroll) {
    if ((t0 & 31) == 0) {  // refill: lane l takes mask word 64*(t0/32)+l of this chunk
      const int w = (t0 >> 5) * 64 + (int)lane;
      held = w < g.W ? mrow[w] : 0u;
    }
    float x[kUnroll];
#pragma unroll
    for (int j = 0; j < kUnroll; j++) {
      const int t = t0 + j;
      const int slot = (2 * t) & 63;
      const uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)held, slot);
      const uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)held, slot + 1);
      unsigned long long m = ((unsigned long long)hi << 32) | lo;
      const int rem = len - t * 64;  // bits past the end of the chunk carry no data
      if (rem < 64) m = rem > 0 ? (m & ((1ull << rem) - 1ull)) : 0ull;
      const bool nz = (m >> lane) & 1ull;
      x[j] = nz ? values[off + rank_below(m)] : 0.0f;
      off += popc64(m);
    }
#pragma unroll
    for (int j = 0; j < kUnroll; j++) {
      const int k = (t0 + j) * 64 + (int)lane;
      if (k < len) q[k] = x[j];
    }
  }
}

// Same expansion with one lane = four consecutive elements and 16-byte stores
// (with the nontemporal hint: 256 MiB expand in 63 instead of 88 us, 32 MiB in
// 10.9 instead of 12.3 us, a reader of the result right after it no slower;
// the same hint on the loads of the counting and compacting passes gains nothing):
// the per-element form above issues one 4-byte store per lane and is bound by
// that instruction stream, not by bytes.  A row is 256 elements = 8 mask words;
// lane l keeps mask word 64*(row/8) + l of the chunk, together with the number
// of set bits in the words before it inside its row, so a lane finds its nibble
// and the rank of its first element with two cross-lane reads.
// Needs E % 4 == 0 and a 16-byte aligned destination (every chunk then starts
// on a 16-byte boundary); the caller checks.
constexpr int kRowsInFlight = 8;  // divides the 8 rows one refill covers

__global__ __launch_bounds__(64 * kWavesPerGroup) void zvc_expand4_kernel(
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
  const int rows = (len + 255) >> 8;
  const unsigned sub = lane & 7u;  // my nibble inside the word I read
  const uint32_t below = (1u << (4u * sub)) - 1u;
  uint32_t held = 0, pre = 0;  // pre: low half = set bits before my word in its row, high half = through it
  for (int r0 = 0; r0 < rows; r0 += kRowsInFlight) {
    {  // refill: 64 words = 8 rows
      const int w = (r0 >> 3) * 64 + (int)lane;
      held = w < g.W ? mrow[w] : 0u;
      const int first = w * 32;  // bits past the end of the chunk carry no data
      if (first + 32 > len) held = first >= len ? 0u : (held & ((1u << (len - first)) - 1u));
      const uint32_t cnt = (uint32_t)__popc(held);
      uint32_t s = cnt;
#pragma unroll
      for (int o = 1; o < 8; o <<= 1) {
        const uint32_t t = (uint32_t)__shfl_up((int)s, o, 64);
        if (sub >= (unsigned)o) s += t;
      }
      pre = (s - cnt) | (s << 16);
    }
    float4 x[kRowsInFlight];
#pragma unroll
    for (int j = 0; j < kRowsInFlight; j++) {
      const int src = (j << 3) + (int)(lane >> 3);
      const uint32_t w = (uint32_t)__shfl((int)held, src, 64);
      const uint32_t p = (uint32_t)__shfl((int)pre, src, 64);
      const uint32_t row_total = (uint32_t)__builtin_amdgcn_readlane((int)pre, (j << 3) + 7) >> 16;
      const uint32_t nib = (w >> (4u * sub)) & 15u;
      unsigned rk = off + (p & 0xffffu) + (unsigned)__popc(w & below);
      float4 v;
      v.x = (nib & 1u) ? values[rk] : 0.0f;
      rk += nib & 1u;
      v.y = (nib & 2u) ? values[rk] : 0.0f;
      rk += (nib >> 1) & 1u;
      v.z = (nib & 4u) ? values[rk] : 0.0f;
      rk += (nib >> 2) & 1u;
      v.w = (nib & 8u) ? values[rk] : 0.0f;
      x[j] = v;
      off += row_total;
    }
#pragma unroll
    for (int j = 0; j < kRowsInFlight; j++) {
      const int k = (r0 + j) * 256 + 4 * (int)lane;
      if (k + 4 <= len) {
        st_stream4(reinterpret_cast<float4*>(q + k), x[j]);
      } else {  // ragged end of the last chunk
        if (k < len) q[k] = x[j].x;
        if (k + 1 < len) q[k + 1] = x[j].y;
        if (k + 2 < len) q[k + 2] = x[j].z;
      }
    }
  }
}

// The same once more for tensors larger than the memory-side cache (the size from which
// the compaction is staged, too): the packed values of four rows (1024 elements) are first
// brought into an LDS region of the wavefront with aligned 16-byte loads -- whole lines per
// instruction -- and picked from there, and the mask words of the next eight rows are asked
// for while the current eight are expanded.  Fetching the values one by one from global
// memory, four partly filled load instructions per row, is 15 % slower where they come from
// HBM (512 MiB: 0.151 against 0.178 ms; staging eight rows at a time 0.167, two 0.163: less
// LDS per wavefront means more wavefronts per compute unit to hide the two loads each group
// waits for, fewer rows per group means more groups) and the same where they come from the
// cache; on small tensors the LDS costs more occupancy than the loads gain, so those keep
// the kernel above.
constexpr int kRowsStaged = 4;  // divides kRowsInFlight

__global__ __launch_bounds__(64 * kWavesPerGroup) void zvc_expand4_staged_kernel(
    const float* __restrict__ values, const uint32_t* __restrict__ mask, const int* __restrict__ begin,
    Geometry g, float* __restrict__ out)
{
  __shared__ __attribute__((aligned(16))) float lds_all[kWavesPerGroup][256 * kRowsStaged + 8];
  const int c = blockIdx.x * kWavesPerGroup + (threadIdx.x >> 6);
  if (c >= g.active) return;
  float* lds = lds_all[threadIdx.x >> 6];
  const unsigned lane = lane_id();
  const long long b = (long long)g.E * c;
  const int len = (int)min((long long)g.E, (long long)g.n - b);
  const uint32_t* mrow = mask + (size_t)c * g.W;
  float* q = out + b;
  unsigned off = (unsigned)begin[c];
  const int rows = (len + 255) >> 8;
  const unsigned sub = lane & 7u;  // my nibble inside the word I read
  const uint32_t below = (1u << (4u * sub)) - 1u;
  uint32_t held_next = (int)lane < g.W ? mrow[lane] : 0u;
  for (int r0 = 0; r0 < rows; r0 += kRowsInFlight) {
    uint32_t held = held_next, pre;  // pre: low half = set bits before my word in its row, high half = through it
    {  // 64 words = 8 rows; the next 64 are asked for now
      const int w = (r0 >> 3) * 64 + (int)lane;
      held_next = w + 64 < g.W ? mrow[w + 64] : 0u;
      const int first = w * 32;  // bits past the end of the chunk carry no data
      if (first + 32 > len) held = first >= len ? 0u : (held & ((1u << (len - first)) - 1u));
      const uint32_t cnt = (uint32_t)__popc(held);
      uint32_t s = cnt;
#pragma unroll
      for (int o = 1; o < 8; o <<= 1) {
        const uint32_t t = (uint32_t)__shfl_up((int)s, o, 64);
        if (sub >= (unsigned)o) s += t;
      }
      pre = (s - cnt) | (s << 16);
    }
#pragma unroll
    for (int h = 0; h < kRowsInFlight; h += kRowsStaged) {
      // where each row's values start inside the group of four, and how many the group has
      unsigned row_start[kRowsStaged], total = 0;
#pragma unroll
      for (int j = 0; j < kRowsStaged; j++) {
        row_start[j] = total;
        total += (uint32_t)__builtin_amdgcn_readlane((int)pre, ((h + j) << 3) + 7) >> 16;
      }
      // values[off, off + total) to lds[shift ...] with loads aligned in global memory (shift = off % 4);
      // the last group of four is fetched element by element so that nothing past the values is read
      const unsigned shift = off & 3u;
      const float* src = values + (off - shift);
      const unsigned end = shift + total;
      lds_order();  // the picks of the previous group are done
      for (unsigned k = 4u * lane; k < end; k += 256u) {
        if (k + 4u <= end) {
          *reinterpret_cast<float4*>(lds + k) = *reinterpret_cast<const float4*>(src + k);
        } else {
          for (unsigned e = k; e < end; e++) lds[e] = src[e];
        }
      }
      lds_order();
      float4 x[kRowsStaged];
#pragma unroll
      for (int j = 0; j < kRowsStaged; j++) {
        const int from = ((h + j) << 3) + (int)(lane >> 3);
        const uint32_t w = (uint32_t)__shfl((int)held, from, 64);
        const uint32_t p = (uint32_t)__shfl((int)pre, from, 64);
        const uint32_t nib = (w >> (4u * sub)) & 15u;
        unsigned rk = shift + row_start[j] + (p & 0xffffu) + (unsigned)__popc(w & below);
        float4 v;
        v.x = (nib & 1u) ? lds[rk] : 0.0f;
        rk += nib & 1u;
        v.y = (nib & 2u) ? lds[rk] : 0.0f;
        rk += (nib >> 1) & 1u;
        v.z = (nib & 4u) ? lds[rk] : 0.0f;
        rk += (nib >> 2) & 1u;
        v.w = (nib & 8u) ? lds[rk] : 0.0f;
        x[j] = v;
      }
      off += total;
#pragma unroll
      for (int j = 0; j < kRowsStaged; j++) {
        const int k = (r0 + h + j) * 256 + 4 * (int)lane;
        if (k + 4 <= len) {
          st_stream4(reinterpret_cast<float4*>(q + k), x[j]);
        } else {  // ragged end of the last chunk
          if (k < len) q[k] = x[j].x;
          if (k + 1 < len) q[k + 1] = x[j].y;
          if (k + 2 < len) q[k + 2] = x[j].z;
        }
      }
    }
  }
}

// ------------------------------------------------------------------ status words
// The single-pass kernel below exchanges counts between workgroups through status words
// in global memory, read and written with relaxed atomics of agent scope (they travel past
// the per-XCD L2 caches, which are not coherent with each other).
// How often a wavefront may ask again for status words it is waiting for, summed over the whole
// kernel (not per word: once the budget is spent every later wait of that wavefront returns at
// once, and a wavefront that sees the failure flag up stops waiting as well, so a run that cannot
// finish -- the grid's workgroups are not all resident at the same time, say -- ends after one
// budget, not after one per tile).  A turn is a sleep and a trip to memory, 1-2 us: the default
// is some tens of milliseconds, two orders of magnitude above what the kernel takes for 1 GiB.
constexpr unsigned kSpinLimit = 1u << 15;
constexpr unsigned kFlagEvery = 32;  // a waiting wavefront looks at the failure flag every so many turns
// cswap_zvc_debug_set_lookback: the bound of the waits, and whether tile 0 is never published
static std::atomic<unsigned> g_spin_limit{kSpinLimit}, g_skip_first{0};

// Head of a workspace.  ws[0]: kWsMagic once cswap_zvc_workspace_clear has prepared it;
// ws[1]: not 0 after a run whose bounded waits ran out (stays until the next clear, and
// every run that finds it reports failure); ws[3]: number of runs whose scanner has
// finished.  The status words proper start at ws[16].  A run that succeeds leaves them
// zero again: whoever consumes a status word clears it.
//
// Who reports what.  The scanner is ahead of everybody else by two stages, so the
// checks and the result are its business and cost the data workgroups nothing: it looks
// at ws[0] and ws[1] when it starts, and when it has published the last offset it writes
// *nnz (the total, or -1 if the flag is up by then) and only then steps ws[3].  A wavefront
// whose wait ran out raises the flag at once; before it ends it waits (bounded) for ws[3]
// to move and then writes -1 itself, so its -1 lands after whatever the scanner wrote, and
// a scanner that is late finds the flag.  A workspace that is refused (never prepared, or
// left behind by a failed run) makes the scanner write -1 and hand out offsets of zero, so
// that every workgroup runs through without waiting; the data workgroups keep every offset
// they are given inside the tensor, whatever the word held.
constexpr uint32_t kWsMagic = 0x5a564331u;
constexpr int kWsFlag = 1, kWsRuns = 3;

__global__ void zvc_ws_clear_kernel(uint32_t* ws, int words)
{
  int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < words) ws[i] = i == 0 ? kWsMagic : 0u;
}

__device__ __forceinline__ uint32_t ld_status(const uint32_t* p)
{
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void st_status(uint32_t* p, uint32_t v)
{
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// ------------------------------------------------------------------ stream
// count + scan + compact in one pass, as a pipeline that never holds data while it
// waits.  The tensor is cut into tiles of 192 rows (a row = 64 elements = two mask
// words); a grid of G resident workgroups (one per compute unit) walks them round
// robin: workgroup w takes tiles w, w+G, w+2G, ...  Each of its sixteen wavefronts keeps
// 12 rows of five consecutive tiles of the workgroup in registers: while tile i is
// compacted, tiles i+1 and i+2 wait counted, tile i+3 is counted and its count published,
// and the loads of tile i+4 are issued one row at a time between the rows of tile i, so
// that memory sees a steady stream of requests instead of bursts.  One more workgroup,
// the scanner, reads the published counts in tile order and publishes each tile's offset;
// a count is published two stages before its tile's offset is needed, which covers the two
// trips through memory (count to the scanner, offset back) that take about a stage each on
// this part, so a workgroup that asks for the offset of its next tile at the start of a
// stage has it when the stage ends, and nobody waits for anybody's latest step.  The
// compacted values go through an LDS stage per tile and leave as whole 16-byte groups
// aligned in the values array.
//
// Needs: chunk length a multiple of 32 (the mask is then the flat bit mask and a chunk
// starts on a half row), two status words per tile in the workspace, a 16-byte aligned
// values pointer, and all G+1 workgroups resident at once (the waits are bounded).
// Workspace (prepared once by cswap_zvc_workspace_clear; a run leaves it as it found it):
// ws[16 + t] = kTileReady | count of tile t, ws[16 + tiles + t] = kTileReady | number of
// non-zeros before tile t; the scanner clears a count when it has read it, a workgroup the
// offsets of its tiles when it is through, so no launch is spent on clearing.
//
// Measured on one MI355X, half of the elements zero (this kernel / count + scan + compact):
// 512 MiB 0.161 / 0.240 ms, 256 MiB 0.082 / 0.115 ms, 128 MiB 0.046 / 0.056, 64 MiB 0.031 /
// 0.033, 32 MiB 0.021 / 0.020 ms (a tensor of a few rounds of the grid does not fill the
// pipeline).
constexpr int kSWaves = 16, kSRows = 12;
constexpr int kSTileRows = kSWaves * kSRows, kSTileElems = kSTileRows * 64;
constexpr int kSSlots = 5;   // tiles of a workgroup in registers
constexpr int kSAhead = kSSlots - 1;  // the loads run this many tiles ahead of the compaction
constexpr uint32_t kTileReady = 1u << 31;

struct StreamGeometry {
  int n, E, process, active;
  int rows;    // rows that exist in the mask layout: process * E / 64 rounded up
  int tiles;   // ceil(rows / 256)
  int mask_words;
};

// Inclusive prefix sum over the 64 lanes of a wavefront with data-parallel-primitive
// moves (row shifts inside rows of 16 lanes, then the row broadcasts): six additions, no
// trip through the LDS crossbar that a shuffle takes.
__device__ __forceinline__ unsigned wave_inclusive_scan(unsigned v)
{
  v += (unsigned)__builtin_amdgcn_update_dpp(0, (int)v, 0x111, 0xf, 0xf, false);  // row_shr:1
  v += (unsigned)__builtin_amdgcn_update_dpp(0, (int)v, 0x112, 0xf, 0xf, false);  // row_shr:2
  v += (unsigned)__builtin_amdgcn_update_dpp(0, (int)v, 0x114, 0xf, 0xf, false);  // row_shr:4
  v += (unsigned)__builtin_amdgcn_update_dpp(0, (int)v, 0x118, 0xf, 0xf, false);  // row_shr:8
  v += (unsigned)__builtin_amdgcn_update_dpp(0, (int)v, 0x142, 0xa, 0xf, false);  // row_bcast:15 into rows 1, 3
  v += (unsigned)__builtin_amdgcn_update_dpp(0, (int)v, 0x143, 0xc, 0xf, false);  // row_bcast:31 into rows 2, 3
  return v;
}

// The scanner: one wavefront turns counts into offsets, 256 tiles at a time, in tile order.
__device__ void zvc_stream_scanner(uint32_t* ws, int tiles, int step, int* nnz, unsigned spin_limit)
{
  if (threadIdx.x >= 64) return;
  const unsigned lane = lane_id();
  uint32_t* status = ws + 16;
  uint32_t* offset = ws + 16 + tiles;
  const uint32_t magic = ld_status(&ws[0]), flag0 = ld_status(&ws[kWsFlag]);
  const bool refused = magic != kWsMagic || flag0 != 0u;
  if (refused && lane == 0) *nnz = -1;
  unsigned carry = 0;
  unsigned spins = 0;    // turns of waiting so far, over all steps
  bool flagged = false;  // the failure flag is up: no more waiting, the offsets from here on are garbage below n
  // `step` tiles at a time (at most 256): the tiles that the data workgroups count in the same
  // stage, so that a step never waits for a count that is published a stage later than the rest
  for (int t0 = 0; t0 < tiles; t0 += step) {
    // lane l owns tiles t0 + 4l .. t0 + 4l + 3
    const int stop = t0 + step < tiles ? t0 + step : tiles;
    uint32_t v[4] = {kTileReady, kTileReady, kTileReady, kTileReady};
    while (!refused) {
      bool missing = false;
#pragma unroll
      for (int r = 0; r < 4; r++) {
        const int t = t0 + 4 * (int)lane + r;
        v[r] = t < stop ? ld_status(&status[t]) : kTileReady;
        missing |= (v[r] & kTileReady) == 0u;
      }
      if (__ballot(missing) == 0ull || flagged) break;
      if (++spins > spin_limit) {  // give up: flag it; the offsets that follow are garbage below n
        if (lane == 0) atomicOr(&ws[kWsFlag], 1u);
        flagged = true;
        break;
      }
      if (spins % kFlagEvery == 0 && ld_status(&ws[kWsFlag]) != 0u) {  // a data workgroup gave up
        flagged = true;
        break;
      }
      __builtin_amdgcn_s_sleep(4);
    }
    // these counts have been read: clear them for the next run
    if (!refused) {
#pragma unroll
      for (int r = 0; r < 4; r++) {
        const int t = t0 + 4 * (int)lane + r;
        if (t < stop) st_status(&status[t], 0u);
      }
    }
    unsigned c[4], mine = 0;
#pragma unroll
    for (int r = 0; r < 4; r++) {
      c[r] = v[r] & ~kTileReady;
      mine += c[r];
    }
    const unsigned incl = wave_inclusive_scan(mine);
    unsigned run = carry + incl - mine;
#pragma unroll
    for (int r = 0; r < 4; r++) {
      const int t = t0 + 4 * (int)lane + r;
      if (t < stop) st_status(&offset[t], kTileReady | run);
      run += c[r];
    }
    carry += (unsigned)__builtin_amdgcn_readlane((int)incl, 63);
  }
  if (lane == 0) {
    if (!refused) *nnz = ld_status(&ws[kWsFlag]) != 0u ? -1 : (int)carry;
    __threadfence();
    __hip_atomic_fetch_add(&ws[kWsRuns], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

template <bool HINT>
__global__ __launch_bounds__(64 * kSWaves) void zvc_stream_kernel(
    const float* __restrict__ in, StreamGeometry g, uint32_t* __restrict__ ws, int* __restrict__ begin,
    int* __restrict__ nnz, float* __restrict__ values, uint32_t* __restrict__ mask, unsigned spin_limit,
    unsigned skip_first)
{
  __shared__ __attribute__((aligned(16))) float stage[kSTileElems + 8];
  __shared__ unsigned s_cnt[kSSlots][kSWaves];
  const int G = (int)gridDim.x - 1, w = (int)blockIdx.x;
  if (w == G) {
    zvc_stream_scanner(ws, g.tiles, G, nnz, spin_limit);
    return;
  }
  const unsigned lane = lane_id();
  const int wv = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  uint32_t* status = ws + 16;
  uint32_t* offset = ws + 16 + g.tiles;
  const int iters = (g.tiles - w + G - 1) / G;  // >= 1: the grid has no more data workgroups than there are tiles
  // chunk index = half row / W by multiply and shift (exact while half rows * W < 2^40)
  const unsigned long long w_magic = ((1ull << 40) + (unsigned)g.E / 32u - 1) / ((unsigned)g.E / 32u);

  float x[kSSlots][kSRows];
  unsigned woff[kSSlots];   // non-zeros of the workgroup's tile in the wavefronts before mine
  unsigned total[kSSlots];  // non-zeros of the workgroup's tile
  // The registers of a slot hold what the loads brought, also for rows that do not exist; `have[slot]`
  // says how many elements do, and whoever looks at the values applies it (a select right after the
  // load would be a use of the value and would make the load's latency part of the stage that issued it).
  int have[kSSlots];
  uint32_t ov = 0;          // the offset word of the workgroup's next tile, once it has arrived (every
                            // wavefront reads it for itself: one more branch-free load per stage)

  // Where my rows of tile t start, as a base that is the same for the whole wavefront and
  // the number of elements that exist from there on (0..768).  Rows that do not exist -- past
  // the end of the tensor, tiles past the last one -- are read from the start of the tensor
  // instead and ignored: every wavefront issues the same loads on every path, so that the
  // compiler's count of loads in flight is exact and a wait for one tile does not also wait
  // for the tile whose loads were issued after it.
  auto rows_of = [&](int t, const float*& base, int& exist) {
    const long long first = ((long long)t * kSTileRows + wv * kSRows) * 64;
    long long left = (long long)g.n - first;
    left = left < 0 ? 0 : (left > kSRows * 64 ? kSRows * 64 : left);
    exist = (int)left;
    base = in + (left > 0 ? first : 0);
  };
  auto count_tile = [&](const float (&src)[kSRows], int slot) {
    unsigned cnt = 0;
    if (have[slot] == kSRows * 64) {
#pragma unroll
      for (int j = 0; j < kSRows; j++) cnt += popc64(__ballot(src[j] != 0.0f));
    } else {
#pragma unroll
      for (int j = 0; j < kSRows; j++) cnt += popc64(__ballot(src[j] != 0.0f && (int)lane < have[slot] - 64 * j));
    }
    if (lane == 0) s_cnt[slot][wv] = cnt;
  };
  // after the barrier that follows count_tile: my offset inside the tile and the tile's total; wave 0 publishes it
  auto share_counts = [&](int slot, int t, bool exists) {
    const unsigned mine = lane < (unsigned)kSWaves ? s_cnt[slot][lane] : 0u;
    const unsigned incl = wave_inclusive_scan(mine);
    total[slot] = (unsigned)__builtin_amdgcn_readlane((int)incl, kSWaves - 1);
    woff[slot] = (unsigned)__builtin_amdgcn_readlane((int)(incl - mine), wv);
    if (wv == 0 && exists && lane == 0 && !(skip_first && t == 0)) st_status(&status[t], kTileReady | total[slot]);
  };
  // waits (bounded) until the scanner has published the offset of tile t
  bool gave_up = false;
  uint32_t runs0 = 0;  // ws[kWsRuns] when this wavefront gave up
  unsigned spins = 0;   // turns of waiting so far, over all tiles
  auto await_offset = [&](int t) {
    while ((ov & kTileReady) == 0u && !gave_up) {
      const bool spent = ++spins > spin_limit;
      if (spent || (spins % kFlagEvery == 0 && ld_status(&ws[kWsFlag]) != 0u)) {
        // give up (my budget is spent, or somebody else's was): flag it and go on with what is
        // there, so that every workgroup still reaches its end (offsets are kept inside the
        // tensor, the output is garbage); no later tile waits again
        if (spent && lane == 0) atomicOr(&ws[kWsFlag], 1u);
        runs0 = ld_status(&ws[kWsRuns]);  // the scanner has not finished: it still owes this offset
        gave_up = true;
        break;
      }
      __builtin_amdgcn_s_sleep(2);
      ov = ld_status(&offset[t]);
    }
  };
  // what the write-out of a tile needs, kept from its scatter to the next stage
  unsigned out_prefix = 0, out_total = 0;
  uint32_t out_held = 0;
  int out_begin_idx = -1, out_begin_val = 0;
  long long out_word = 0;
  unsigned prev_prefix = 0, prev_total = 0;
  auto write_out = [&](unsigned tile_prefix, unsigned tile_total) {
    const unsigned shift = tile_prefix & 3u;
    const unsigned end = shift + tile_total;           // stage slots [shift, end) hold data
    float* base = values + (tile_prefix - shift);      // 16-byte aligned
    for (unsigned q = threadIdx.x; 4u * q < end; q += 64 * kSWaves) {
      const stream_f4 v = *reinterpret_cast<const stream_f4*>(stage + 4u * q);
      float* dst = base + 4u * q;
      if (4u * q >= shift && 4u * q + 4u <= end) {
        if (HINT) __builtin_nontemporal_store(v, reinterpret_cast<stream_f4*>(dst));
        else *reinterpret_cast<stream_f4*>(dst) = v;
      } else {  // the first and the last group of a tile are shared with its neighbours
        if (4u * q + 0u >= shift && 4u * q + 0u < end) dst[0] = v.x;
        if (4u * q + 1u >= shift && 4u * q + 1u < end) dst[1] = v.y;
        if (4u * q + 2u >= shift && 4u * q + 2u < end) dst[2] = v.z;
        if (4u * q + 3u >= shift && 4u * q + 3u < end) dst[3] = v.w;
      }
    }
    if (lane < 2u * kSRows && out_word < (long long)g.mask_words) mask[out_word] = out_held;
    if (out_begin_idx >= 0) begin[out_begin_idx] = out_begin_val;
  };

  // ---- fill the pipeline: four tiles on their way, the first three counted and published
  {
    const float* base;
    int exist;
#pragma unroll
    for (int k = 0; k < kSAhead; k++) {
      rows_of(w + k * G, base, exist);
      have[k] = exist;
#pragma unroll
      for (int j = 0; j < kSRows; j++) x[k][j] = base[min(lane + 64u * j, (unsigned)max(exist - 1, 0))];
    }
  }
#pragma unroll
  for (int k = 0; k < kSAhead - 1; k++) count_tile(x[k], k);
  __syncthreads();
#pragma unroll
  for (int k = 0; k < kSAhead - 1; k++) share_counts(k, w + k * G, k < iters);
  ov = ld_status(&offset[w]);

  for (int i0 = 0; i0 < iters; i0 += kSSlots) {
#pragma unroll
    for (int s = 0; s < kSSlots; s++) {
      const int i = i0 + s;
      if (i >= iters) break;
      const int t = i * G + w;
      // ---- this tile's offset was asked for a stage ago; ask for the next one
      await_offset(t);
      out_total = total[s];
      // whatever the word held (a workspace that was never prepared, a wait that ran out): what this
      // tile writes stays inside the tensor
      // (in a vector register on purpose: as a scalar the compiler fetches the word's value the
      // moment it was asked for, which waits for every load in flight)
      {
        uint32_t given = ov & ~kTileReady;
        asm volatile("" : "+v"(given));
        out_prefix = min(given, (unsigned)g.n - out_total);
      }
      // ---- the previous tile leaves
      if (i > 0) write_out(prev_prefix, prev_total);
      prev_prefix = out_prefix;
      prev_total = out_total;
      __syncthreads();
      ov = ld_status(&offset[i + 1 < iters ? t + G : t]);
      // ---- non-zeros of this tile into the LDS stage, one row at a time, and after each row the
      // load of the same row of the tile four ahead, so that the requests to memory are spread
      // over the whole stage instead of arriving in a burst
      {
        const int r0 = t * kSTileRows + wv * kSRows;  // my first row
        unsigned at = (out_prefix & 3u) + woff[s];    // stage slot of the next non-zero
        const unsigned at0 = at;
        uint32_t held = 0;
        const float* base;
        int exist;
        rows_of(t + kSAhead * G, base, exist);
        have[(s + kSAhead) % kSSlots] = exist;
        const unsigned last = (unsigned)max(exist - 1, 0);
        // the same loop twice: with every row of both tiles there (nearly always), and with the checks
        // for rows that are not; both issue the same twelve loads
        if (have[s] == kSRows * 64 && exist == kSRows * 64) {
#pragma unroll
          for (int j = 0; j < kSRows; j++) {
            const float v = x[s][j];
            const bool nz = v != 0.0f;
            const unsigned long long m = __ballot(nz);
            const unsigned slot =
                __builtin_amdgcn_mbcnt_hi((unsigned)(m >> 32), __builtin_amdgcn_mbcnt_lo((unsigned)m, at));
            if (nz) stage[slot] = v;
            at += popc64(m);
            if (lane == 2u * j) held = (uint32_t)m;
            if (lane == 2u * j + 1u) held = (uint32_t)(m >> 32);
            x[(s + kSAhead) % kSSlots][j] = base[lane + 64u * j];
          }
        } else {
#pragma unroll
          for (int j = 0; j < kSRows; j++) {
            const float v = x[s][j];
            const bool nz = v != 0.0f && (int)lane < have[s] - 64 * j;
            const unsigned long long m = __ballot(nz);
            const unsigned slot =
                __builtin_amdgcn_mbcnt_hi((unsigned)(m >> 32), __builtin_amdgcn_mbcnt_lo((unsigned)m, at));
            if (nz) stage[slot] = v;
            at += popc64(m);
            if (lane == 2u * j) held = (uint32_t)m;
            if (lane == 2u * j + 1u) held = (uint32_t)(m >> 32);
            x[(s + kSAhead) % kSSlots][j] = base[min(lane + 64u * j, last)];
          }
        }
        // lane k < 32 holds mask word k of my rows = half row 2*r0 + k; a chunk starts there
        // if the half row index is a multiple of W
        const unsigned in_word = (unsigned)__popc(held);
        const unsigned before = wave_inclusive_scan(in_word) - in_word;
        const unsigned half = 2u * (unsigned)r0 + lane;
        const unsigned c = (unsigned)(((unsigned long long)half * w_magic) >> 40);
        const bool starts = lane < 2u * kSRows && c * ((unsigned)g.E / 32u) == half && (int)c < g.active;
        out_begin_idx = starts ? (int)c : -1;
        out_begin_val = (int)(out_prefix - (out_prefix & 3u) + at0 + before);
        out_held = held;
        out_word = (long long)r0 * 2 + lane;
      }
      // ---- the tile three ahead arrived during the previous stage: count it (in the same
      // straight line as the loads above, so that the wait for it knows which loads are younger)
      count_tile(x[(s + kSAhead - 1) % kSSlots], (s + kSAhead - 1) % kSSlots);
      __syncthreads();
      share_counts((s + kSAhead - 1) % kSSlots, t + (kSAhead - 1) * G, i + kSAhead - 1 < iters);
    }
  }
  write_out(prev_prefix, prev_total);
  // ---- the offsets of my tiles have all been read: clear them for the next run (here and not tile by
  // tile: a store per stage from one wavefront, small as it is, costs the pipeline 4 % at 256 MiB)
  for (int i = (int)threadIdx.x; i < iters; i += 64 * kSWaves) st_status(&offset[i * G + w], 0u);
  // ---- a wavefront whose wait ran out says so after the scanner has written its result
  if (gave_up) {
    for (unsigned spins = 0; ld_status(&ws[kWsRuns]) == runs0 && spins < spin_limit; spins++)
      __builtin_amdgcn_s_sleep(2);
    if (lane == 0) *nnz = -1;
  }
}

// ------------------------------------------------------------------ one kernel for small tensors
// Up to 32 MiB the whole tensor fits in the registers of one grid: every workgroup (one per
// compute unit, sixteen wavefronts) loads its share once -- wavefront v of workgroup w owns R
// consecutive rows of 64 elements --, counts it, writes its mask words, and publishes its count.
// There is no scanner: every workgroup reads the counts of the workgroups before it itself, one
// trip through memory instead of two, takes their sum as its offset, and stores its non-zeros
// straight from the registers (at these sizes the values array stays in the memory-side cache,
// where whole-line stores through an LDS stage gain nothing).  The last workgroup, which has
// read every count but its own, writes the total.  Nobody waits for a workgroup with a higher
// number than its own, so the grid makes progress however few of its workgroups the hardware
// runs at a time (they are started in order).
//
// The counts live in two arrays of 256 words at the end of the workspace, used in turns: run
// k publishes into array k & 1 and every workgroup clears its word of the other one, which
// nobody reads any more; ws[kWsSmallRuns] counts the runs.  The grid is the same for every
// size, so every word is cleared every time.  Failure works as in the pipeline kernel: a wait
// that runs out raises the sticky flag, the offsets are kept inside the tensor, and the
// wavefront that gave up writes -1 after the last workgroup has stepped the run counter.
constexpr int kQWaves = 16;
constexpr int kQGroupsMax = 256;
constexpr int kWsSmallRuns = 4;
constexpr int kSmallWords = 2 * kQGroupsMax;  // taken from the end of the workspace's status words

template <int R>
__global__ __launch_bounds__(64 * kQWaves) void zvc_small_kernel(
    const float* __restrict__ in, StreamGeometry g, uint32_t* __restrict__ ws, uint32_t* __restrict__ counts,
    int* __restrict__ begin, int* __restrict__ nnz, float* __restrict__ values, uint32_t* __restrict__ mask,
    unsigned spin_limit, unsigned skip_first)
{
  constexpr int kHeld = (R + 31) / 32;  // registers of mask words: lane l of register h holds half row 64h + l
  __shared__ unsigned s_cnt[kQWaves];
  __shared__ unsigned s_head[4];        // refused, parity, my offset, total
  const int G = (int)gridDim.x, w = (int)blockIdx.x;
  const unsigned lane = lane_id();
  const int wv = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const int r0 = (w * kQWaves + wv) * R;  // my first row

  // ---- my rows; rows that do not exist are read from the start of the tensor and ignored
  const long long first = (long long)r0 * 64;
  long long left_ll = (long long)g.n - first;
  left_ll = left_ll < 0 ? 0 : (left_ll > R * 64 ? R * 64 : left_ll);
  const int left = (int)left_ll;
  const float* base = in + (left > 0 ? first : 0);
  const unsigned last = (unsigned)max(left - 1, 0);
  float x[R];
#pragma unroll
  for (int j = 0; j < R; j++) x[j] = base[min(lane + 64u * j, last)];
  if (threadIdx.x == 0) {  // together with the data: is the workspace usable, and which count array is this run's
    const uint32_t magic = ld_status(&ws[0]), flag = ld_status(&ws[kWsFlag]), runs = ld_status(&ws[kWsSmallRuns]);
    s_head[0] = (magic != kWsMagic || flag != 0u) ? 1u : 0u;
    s_head[1] = runs;
  }

  // ---- count, and the mask words (two per row, straight from the ballots)
  unsigned cnt = 0;
  uint32_t held[kHeld];
#pragma unroll
  for (int h = 0; h < kHeld; h++) held[h] = 0;
#pragma unroll
  for (int j = 0; j < R; j++) {
    const unsigned long long m = __ballot(x[j] != 0.0f && (int)lane < left - 64 * j);
    cnt += popc64(m);
    if (lane == 2u * (j % 32)) held[j / 32] = (uint32_t)m;
    if (lane == 2u * (j % 32) + 1u) held[j / 32] = (uint32_t)(m >> 32);
  }
#pragma unroll
  for (int h = 0; h < kHeld; h++) {
    const long long word = ((long long)r0 + 32 * h) * 2 + lane;
    if ((int)lane < 2 * (R - 32 * h) && word < (long long)g.mask_words) mask[word] = held[h];
  }
  if (lane == 0) s_cnt[wv] = cnt;
  __syncthreads();
  if (s_head[0] != 0u) {  // refused: nothing is published, nothing written but the result
    if (w == 0 && threadIdx.x == 0) *nnz = -1;
    return;
  }
  const uint32_t runs0 = s_head[1];
  uint32_t* mine_arr = counts + (runs0 & 1u) * kQGroupsMax;
  const unsigned wave_cnt = lane < (unsigned)kQWaves ? s_cnt[lane] : 0u;
  const unsigned wave_incl = wave_inclusive_scan(wave_cnt);
  const unsigned group_total = (unsigned)__builtin_amdgcn_readlane((int)wave_incl, kQWaves - 1);
  const unsigned woff = (unsigned)__builtin_amdgcn_readlane((int)(wave_incl - wave_cnt), wv);
  if (threadIdx.x == 0) {
    st_status(&counts[((runs0 & 1u) ^ 1u) * kQGroupsMax + w], 0u);
    if (!(skip_first && w == 0)) st_status(&mine_arr[w], kTileReady | group_total);
  }

  // ---- wavefront 0 collects the counts of the workgroups before this one: lane l looks at workgroups 4l .. 4l+3
  bool gave_up = false;
  if (wv == 0) {
    uint32_t v[4];
    unsigned spins = 0;
    for (;;) {
      bool missing = false;
#pragma unroll
      for (int r = 0; r < 4; r++) {
        const int k = 4 * (int)lane + r;
        v[r] = k < w ? ld_status(&mine_arr[k]) : kTileReady;
        missing |= (v[r] & kTileReady) == 0u;
      }
      if (__ballot(missing) == 0ull) break;
      if (++spins > spin_limit) {
        if (lane == 0) atomicOr(&ws[kWsFlag], 1u);
        gave_up = true;
        break;
      }
      __builtin_amdgcn_s_sleep(2);
    }
    unsigned c[4], lane_sum = 0;
#pragma unroll
    for (int r = 0; r < 4; r++) {
      c[r] = v[r] & ~kTileReady;
      lane_sum += c[r];
    }
    const unsigned incl = wave_inclusive_scan(lane_sum);
    // counts of the workgroups before mine: whole lanes below lane w/4, and the first w%4 of that lane
    unsigned part = incl - lane_sum;
#pragma unroll
    for (int r = 0; r < 3; r++) part += r < (w & 3) ? c[r] : 0u;
    const unsigned before_me = (unsigned)__builtin_amdgcn_readlane((int)part, w >> 2);
    const unsigned total = (unsigned)__builtin_amdgcn_readlane((int)incl, 63) + group_total;  // the last workgroup's is the tensor's
    if (lane == 0) {
      // whatever the words held: what this workgroup writes stays inside the tensor
      s_head[2] = min(before_me, (unsigned)g.n - group_total);
      s_head[3] = total;
    }
  }
  __syncthreads();
  uint32_t flag_late = 0;
  if (w == G - 1 && threadIdx.x == 0) flag_late = ld_status(&ws[kWsFlag]);  // asked for now, looked at when the rows are out

  // ---- my non-zeros, row by row, straight from the lanes that hold them; chunk starts on the way
  unsigned at = s_head[2] + woff;
  const unsigned long long w_magic = ((1ull << 40) + (unsigned)g.E / 32u - 1) / ((unsigned)g.E / 32u);
#pragma unroll
  for (int h = 0; h < kHeld; h++) {
    const unsigned in_word = (unsigned)__popc(held[h]);
    const unsigned before = wave_inclusive_scan(in_word) - in_word;
    const unsigned half = 2u * ((unsigned)r0 + 32u * h) + lane;
    const unsigned c = (unsigned)(((unsigned long long)half * w_magic) >> 40);
    if ((int)lane < 2 * (R - 32 * h) && c * ((unsigned)g.E / 32u) == half && (int)c < g.active)
      begin[c] = (int)(at + before);
#pragma unroll
    for (int j = 32 * h; j < R && j < 32 * h + 32; j++) {
      const float v = x[j];
      const bool nz = v != 0.0f && (int)lane < left - 64 * j;
      const unsigned long long m = __ballot(nz);
      if (nz) values[at + rank_below(m)] = v;
      at += popc64(m);
    }
  }

  // ---- the result
  if (w == G - 1 && threadIdx.x == 0) {
    *nnz = (gave_up || flag_late != 0u) ? -1 : (int)s_head[3];
    __threadfence();
    __hip_atomic_fetch_add(&ws[kWsSmallRuns], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  } else if (gave_up && w != G - 1) {  // (wavefront 0 of another workgroup) after the last workgroup has spoken
    for (unsigned spins = 0; ld_status(&ws[kWsSmallRuns]) == runs0 && spins < spin_limit; spins++)
      __builtin_amdgcn_s_sleep(2);
    if (lane == 0) *nnz = -1;
  }
}

// ------------------------------------------------------------------ probe
__global__ void zero_u64_kernel(unsigned long long* p) { *p = 0ull; }

__global__ __launch_bounds__(1024) void probe_nnz_kernel(const float* __restrict__ in, size_t n,
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
  size_t i = tid;
  for (; i + 3 * nthreads < n4; i += 4 * nthreads) {  // four independent 16-byte loads in flight per lane
    float4 v0 = p4[i], v1 = p4[i + nthreads], v2 = p4[i + 2 * nthreads], v3 = p4[i + 3 * nthreads];
    acc += (v0.x != 0.0f) + (v0.y != 0.0f) + (v0.z != 0.0f) + (v0.w != 0.0f);
    acc += (v1.x != 0.0f) + (v1.y != 0.0f) + (v1.z != 0.0f) + (v1.w != 0.0f);
    acc += (v2.x != 0.0f) + (v2.y != 0.0f) + (v2.z != 0.0f) + (v2.w != 0.0f);
    acc += (v3.x != 0.0f) + (v3.y != 0.0f) + (v3.z != 0.0f) + (v3.w != 0.0f);
  }
  for (; i < n4; i += nthreads) {
    float4 v = p4[i];
    acc += (v.x != 0.0f) + (v.y != 0.0f) + (v.z != 0.0f) + (v.w != 0.0f);
  }
  for (size_t i = head + (n4 << 2) + tid; i < n; i += nthreads) acc += (in[i] != 0.0f);
  acc = (unsigned)wave_sum((int)acc);
  // one atomic per workgroup, and few workgroups: same-address atomics from
  // different XCDs serialise at the memory side (~12 ns each)
  __shared__ unsigned part[16];
  if ((threadIdx.x & 63u) == 0) part[threadIdx.x >> 6] = acc;
  __syncthreads();
  if (threadIdx.x == 0) {
    unsigned long long s = 0;
    for (unsigned w = 0; w < (blockDim.x >> 6); w++) s += part[w];
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
  g.backwards = n > (48 << 20);  // more than 192 MB of fp32
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

extern "C" size_t cswap_zvc_set_staged_compact_bytes(size_t bytes)
{
  return (size_t)g_staged_compact_bytes.exchange(bytes);
}

extern "C" int cswap_zvc_compact(const float* d_in, int n, int process, const int* d_begin, float* d_values,
                                 uint32_t* d_mask, cswap_stream_t stream)
{
  if (!d_in || !d_begin || !d_values || !d_mask) return CSWAP_E_ARG;
  Geometry g;
  int rc = make_geometry(g, n, process);
  if (rc) return rc;
  unsigned grid = (g.process + kWavesPerGroup - 1) / kWavesPerGroup;
  if ((reinterpret_cast<uintptr_t>(d_values) & 15u) == 0 && 4ull * (unsigned long long)n >= g_staged_compact_bytes)
    hipLaunchKernelGGL(zvc_compact_kernel, dim3(grid), dim3(64 * kWavesPerGroup), 0, (hipStream_t)stream, d_in,
                       g, d_begin, d_values, d_mask);
  else
    hipLaunchKernelGGL(zvc_compact_rows_kernel, dim3(grid), dim3(64 * kWavesPerGroup), 0, (hipStream_t)stream,
                       d_in, g, d_begin, d_values, d_mask);
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
  const bool quads = g.E % 4 == 0 && (reinterpret_cast<uintptr_t>(d_out) & 15u) == 0;
  if (quads && (reinterpret_cast<uintptr_t>(d_values) & 15u) == 0 &&
      4ull * (unsigned long long)n >= g_staged_compact_bytes)
    hipLaunchKernelGGL(zvc_expand4_staged_kernel, dim3(grid), dim3(64 * kWavesPerGroup), 0, (hipStream_t)stream,
                       d_values, d_mask, d_begin, g, d_out);
  else if (quads)
    hipLaunchKernelGGL(zvc_expand4_kernel, dim3(grid), dim3(64 * kWavesPerGroup), 0, (hipStream_t)stream,
                       d_values, d_mask, d_begin, g, d_out);
  else
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

// Chunk count for a tensor of n elements when the caller is free to choose:
// about 1024 elements per chunk, as a power of two between 1024 and 16384.
// Measured on one MI355X (count + scan + compact, then expand, half-zero data):
// 1 and 4 MiB tensors run 40 % / 60 % faster with 1024 chunks than with the
// reference's 16384, 16 MiB is best at 4096, 32 MiB at 8192, 128 MiB and above
// at 16384 and more; below ~1000 elements per chunk the wavefronts are too short
// to cover their start-up, above ~4000 too few are in flight.
extern "C" int cswap_zvc_pick_process(size_t n)
{
  size_t target = n / 1024;
  int p = 1024;
  while (p < 16384 && (size_t)p * 2 <= target) p *= 2;
  return p;
}

constexpr int kStatusWordsMin = 65536;
// status words of a workspace for `process` chunks: one per chunk for the look-back kernel,
// one per tile for the pipeline kernel, never fewer than 65536
static int status_words(int process) { return process > kStatusWordsMin ? process : kStatusWordsMin; }

extern "C" size_t cswap_zvc_workspace_bytes(int process)
{
  return process > 0 ? ((size_t)status_words(process) + 16) * sizeof(uint32_t) : 0;
}

extern "C" void cswap_zvc_debug_set_lookback(unsigned spin_limit, unsigned skip_first)
{
  g_spin_limit.store(spin_limit ? spin_limit : kSpinLimit);
  g_skip_first.store(skip_first);
}

static int status_words(int process);
// Tensors of at least this many bytes take the single pass in cswap_zvc_compress_fused; smaller ones
// finish sooner with the three kernels (a few rounds of the grid do not fill the pipeline).
static std::atomic<unsigned long long> g_single_pass_bytes{64ull << 20};  // cswap_zvc_set_single_pass_bytes

extern "C" size_t cswap_zvc_set_single_pass_bytes(size_t bytes)
{
  return (size_t)g_single_pass_bytes.exchange(bytes);
}

// Data workgroups of the pipeline kernel: one per compute unit but one (the scanner's), no more
// than there are tiles, and no more than the 256 tiles whose counts the scanner's one wavefront
// turns into offsets per step (four per lane) -- on a part with more compute units than that the
// tiles past the 256th of every step would never get an offset.
static int stream_data_groups(int tiles, int compute_units)
{
  int g = compute_units - 1;
  if (g > tiles) g = tiles;
  if (g > 4 * 64) g = 4 * 64;
  return g < 0 ? 0 : g;
}
extern "C" int cswap_test_zvc_stream_groups(int tiles, int compute_units) { return stream_data_groups(tiles, compute_units); }

// whether the single pass takes a tensor of this shape; fills its geometry
static bool single_pass_shape(const Geometry& g, int n, int process, StreamGeometry& sg)
{
  sg.n = n; sg.E = g.E; sg.process = process; sg.active = g.active;
  const long long mask_words = (long long)g.W * process;
  sg.mask_words = (int)mask_words;
  sg.rows = (int)((mask_words + 1) / 2);
  sg.tiles = (sg.rows + kSTileRows - 1) / kSTileRows;
  // whole half rows per chunk, two status words per tile in the workspace, a compute unit for
  // every workgroup, and a tensor large enough to fill the pipeline
  return g.E % 32 == 0 && mask_words < (1ll << 31) - 64 && 2 * sg.tiles <= status_words(process) - kSmallWords &&
         device_compute_units() > 1 && 4ull * (unsigned long long)n >= g_single_pass_bytes;
}

// Whether the one-kernel form for small tensors takes this shape (a tensor below the size from
// which the pipeline kernel runs, whole half rows per chunk, the whole tensor in the registers
// of one grid); fills the geometry, the grid and the rows per wavefront.
static bool small_pass_shape(const Geometry& g, int n, int process, StreamGeometry& sg, int* groups, int* rows_per_wave)
{
  sg.n = n; sg.E = g.E; sg.process = process; sg.active = g.active;
  const long long mask_words = (long long)g.W * process;
  sg.mask_words = (int)mask_words;
  sg.rows = (int)((mask_words + 1) / 2);
  sg.tiles = 0;
  const int cus = device_compute_units();
  const int G = cus < kQGroupsMax ? cus : kQGroupsMax;
  const unsigned long long single_from = g_single_pass_bytes.load();
  if (G < 1 || g.E % 32 != 0 || single_from == ~0ull || 4ull * (unsigned long long)n >= single_from) return false;
  // every row of the mask layout has an owner, also the rows of chunks that hold no data (their words are zero)
  int R = 8;  // 8, 16 or 32 rows per wavefront (64 would need more registers than a wavefront of sixteen has)
  while (R <= 32 && (long long)G * kQWaves * R < (long long)sg.rows) R *= 2;
  if (R > 32) return false;
  *groups = G;
  *rows_per_wave = R;
  return true;
}

extern "C" int cswap_zvc_takes_single_pass(int n, int process)
{
  Geometry g;
  StreamGeometry sg;
  int groups, rows;
  if (make_geometry(g, n, process) != CSWAP_OK) return 0;
  if (single_pass_shape(g, n, process, sg)) return 1;
  return small_pass_shape(g, n, process, sg, &groups, &rows) ? 2 : 0;
}

extern "C" int cswap_zvc_compress_fused(const float* d_in, int n, int process, void* d_ws, int* d_begin,
                                        int* d_nnz, float* d_values, uint32_t* d_mask, cswap_stream_t stream)
{
  if (!d_in || !d_ws || !d_begin || !d_nnz || !d_values || !d_mask) return CSWAP_E_ARG;
  Geometry g;
  int rc = make_geometry(g, n, process);
  if (rc) return rc;
  uint32_t* ws = (uint32_t*)d_ws;
  const int cus = device_compute_units();
  StreamGeometry sg;
  // anything the single pass does not take, or an output that is not 16-byte aligned, runs the three kernels
  const bool single_pass = single_pass_shape(g, n, process, sg) && (reinterpret_cast<uintptr_t>(d_values) & 15u) == 0;
  int groups = 0, rows = 0;
  if (!single_pass && small_pass_shape(g, n, process, sg, &groups, &rows)) {
    uint32_t* counts = ws + 16 + status_words(process) - kSmallWords;
#define CSWAP_SMALL(R)                                                                                              \
  hipLaunchKernelGGL(zvc_small_kernel<R>, dim3(groups), dim3(64 * kQWaves), 0, (hipStream_t)stream, d_in, sg, ws, \
                     counts, d_begin, d_nnz, d_values, d_mask, g_spin_limit.load(), g_skip_first.load())
    if (rows == 8) CSWAP_SMALL(8);
    else if (rows == 16) CSWAP_SMALL(16);
    else CSWAP_SMALL(32);
#undef CSWAP_SMALL
    return check_launch();
  }
  if (!single_pass) return cswap_zvc_compress(d_in, n, process, d_begin, d_nnz, d_values, d_mask, stream);
  // one workgroup per compute unit, the last of them the scanner
  const int data_groups = stream_data_groups(sg.tiles, cus);
  if (4ull * (unsigned long long)n >= g_staged_compact_bytes)
    hipLaunchKernelGGL(zvc_stream_kernel<true>, dim3(data_groups + 1), dim3(64 * kSWaves), 0, (hipStream_t)stream,
                       d_in, sg, ws, d_begin, d_nnz, d_values, d_mask, g_spin_limit.load(), g_skip_first.load());
  else
    hipLaunchKernelGGL(zvc_stream_kernel<false>, dim3(data_groups + 1), dim3(64 * kSWaves), 0, (hipStream_t)stream,
                       d_in, sg, ws, d_begin, d_nnz, d_values, d_mask, g_spin_limit.load(), g_skip_first.load());
  return check_launch();
}

// ------------------------------------------------------------------ no allocation
// The single-pass compression once more, for callers that cannot bring a workspace
// because they cannot allocate one: the status words live in this array, one copy
// per GPU, held until the process ends.
constexpr int kStaticProcessMax = 65536;
static __device__ __align__(256) uint32_t scratch[kStaticProcessMax + 16] = {kWsMagic};  // prepared from the start

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
uint32_t* g_scratch_ptr[kMaxDevices];  // device address of `scratch` on each GPU, once looked up
}  // namespace

// device address of this GPU's copy of `scratch` (looked up on first use), or an error code
static int static_workspace(uint32_t** ws)
{
  int dev = -1;
  CSWAP_HIP_TRY(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDevices) return CSWAP_E_UNSUPPORTED;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {  // first call on this GPU: where its copy of the array lives
    void* p = nullptr;
    CSWAP_HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    g_scratch_ptr[dev] = static_cast<uint32_t*>(p);
  }
  *ws = g_scratch_ptr[dev];
  return CSWAP_OK;
}

extern "C" int cswap_zvc_compress_fused_static(const float* d_in, int n, int process, int* d_begin, int* d_nnz,
                                               float* d_values, uint32_t* d_mask, cswap_stream_t stream)
{
  if (process > kStaticProcessMax) return CSWAP_E_NOMEM;
  uint32_t* ws = nullptr;
  int rc = static_workspace(&ws);
  if (rc) return rc;
  return cswap_zvc_compress_fused(d_in, n, process, ws, d_begin, d_nnz, d_values, d_mask, stream);
}

extern "C" int cswap_zvc_workspace_clear(void* d_ws, int process, cswap_stream_t stream)
{
  uint32_t* ws = static_cast<uint32_t*>(d_ws);
  if (!ws) {  // the static array of the current GPU
    int rc = static_workspace(&ws);
    if (rc) return rc;
    process = kStaticProcessMax;
  }
  if (process <= 0) return CSWAP_E_ARG;
  const int words = status_words(process) + 16;
  hipLaunchKernelGGL(zvc_ws_clear_kernel, dim3((words + 255) / 256), dim3(256), 0, (hipStream_t)stream, ws, words);
  return check_launch();
}

extern "C" int cswap_probe_nnz(const float* d_in, size_t n, unsigned long long* d_nnz, cswap_stream_t stream)
{
  if (!d_in || !d_nnz || !n) return CSWAP_E_ARG;
  hipLaunchKernelGGL(zero_u64_kernel, dim3(1), dim3(1), 0, (hipStream_t)stream, d_nnz);
  size_t want = (n / 16 + 1023) / 1024;  // 4 float4 per thread and pass
  unsigned grid = (unsigned)(want < 1 ? 1 : (want > 512 ? 512 : want));
  hipLaunchKernelGGL(probe_nnz_kernel, dim3(grid), dim3(1024), 0, (hipStream_t)stream, d_in, n, d_nnz);
  return check_launch();
}
