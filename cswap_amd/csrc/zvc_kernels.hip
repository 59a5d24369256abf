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

#include <mutex>

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
static unsigned long long g_staged_compact_bytes = CSWAP_STAGED_COMPACT_BYTES;  // cswap_zvc_set_staged_compact_bytes

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

// ------------------------------------------------------------------ fused
// count + scan + compact in ONE pass over the tensor: a wavefront keeps its whole
// chunk in registers (IT values per lane) and counts it; the WAVES chunks of a
// workgroup form a tile whose exclusive offset comes from a decoupled look-back
// over tile-granular status words; then every wave writes mask and packed values
// from its registers.  HBM traffic is the algorithmic 4 + 1/8 + 4d bytes per
// element.  Tiles (not chunks) are the unit of the look-back, and one memory
// round trip covers a window of 256 tiles, because a workgroup that starts while
// thousands of others are in flight has to walk back over all of them.
//
// Workspace (zeroed by zvc_ws_zero_kernel before every launch):
//   ws[0]  ticket counter: tiles are handed out in the order workgroups start,
//          so every tile a workgroup waits for belongs to a workgroup that is
//          already running (no dependence on the dispatch order)
//   ws[1]  error flag: set if a bounded wait ran out (never in a healthy run);
//          the same event stores -1 in *nnz, which is what the caller sees
//   ws[16 + t]  status of tile t: bits 31..30 = 0 nothing yet, 1 = count of the
//          tile alone, 2 = inclusive prefix; bits 29..0 = the value
constexpr uint32_t kFlagAgg = 1u << 30, kFlagPre = 2u << 30, kValMask = (1u << 30) - 1u;
constexpr unsigned kSpinLimit = 1u << 22;
// cswap_zvc_debug_set_lookback: the bound of the wait and the first ticket handed out
static unsigned g_spin_limit = kSpinLimit, g_first_ticket = 0;

// Clears the workspace, sets the ticket counter and arms *nnz: the tile that ends
// the tensor lowers it to the total with atomicMin, a wait that ran out lowers it to -1,
// so -1 wins whichever comes first.
__global__ void zvc_ws_zero_kernel(uint32_t* ws, int words, uint32_t first_ticket, int* nnz)
{
  int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < words) ws[i] = i == 0 ? first_ticket : 0u;
  if (i == 0) *nnz = 0x7fffffff;
}

__device__ __forceinline__ uint32_t ld_status(const uint32_t* p)
{
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void st_status(uint32_t* p, uint32_t v)
{
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

template <int IT, int WAVES>
__global__ __launch_bounds__(64 * WAVES) void zvc_fused_kernel(
    const float* __restrict__ in, Geometry g, uint32_t* __restrict__ ws, int* __restrict__ begin,
    int* __restrict__ nnz, float* __restrict__ values, uint32_t* __restrict__ mask, unsigned spin_limit)
{
  __shared__ unsigned s_agg[WAVES];
  __shared__ unsigned s_tile;   // ticket, then the tile's exclusive offset
  const unsigned lane = lane_id();
  const int wv = (int)(threadIdx.x >> 6);
  uint32_t* status = ws + 16;
  if (threadIdx.x == 0) s_tile = atomicAdd(&ws[0], 1u);
  __syncthreads();
  const int tile = (int)s_tile;
  if (tile >= (int)gridDim.x) return;  // only when the ticket counter did not start at zero
  const int c = tile * WAVES + wv;
  const bool in_layout = c < g.process;
  const bool has_data = c < g.active;

  const long long b = (long long)g.E * c;
  const int len = has_data ? (int)min((long long)g.E, (long long)g.n - b) : 0;
  const float* p = in + b;
  const int iters = (g.E + 63) >> 6;  // <= IT

  // ---- phase 1: the chunk into registers, and its count
  float x[IT];
#pragma unroll
  for (int t = 0; t < IT; t++) {
    const int k = t * 64 + (int)lane;
    x[t] = (t < iters && k < len) ? p[k] : 0.0f;
  }
  unsigned agg = 0;
#pragma unroll
  for (int t = 0; t < IT; t++) agg += popc64(__ballot(x[t] != 0.0f));
  if (lane == 0) s_agg[wv] = agg;
  __syncthreads();  // also orders the read of the ticket before s_tile is reused

  // ---- wave 0: decoupled look-back over the tiles before this one
  if (wv == 0) {
    unsigned tile_agg = 0;
#pragma unroll
    for (int w = 0; w < WAVES; w++) tile_agg += s_agg[w];
    unsigned excl = 0;
    if (tile == 0) {
      if (lane == 0) st_status(&status[0], kFlagPre | tile_agg);
    } else {
      if (lane == 0) st_status(&status[tile], kFlagAgg | tile_agg);
      int idx = tile - 1;
      bool done = false;
      while (!done) {
        // one round trip fetches a window of 256 predecessors (4 per lane)
        uint32_t v[4];
        unsigned spins = 0;
        for (;;) {
          bool missing = false;
#pragma unroll
          for (int r = 0; r < 4; r++) {
            const int j = idx - 64 * r - (int)lane;
            v[r] = j >= 0 ? ld_status(&status[j]) : kFlagPre;  // before the first tile: prefix 0
            missing |= (v[r] >> 30) == 0u;
          }
          if (__ballot(missing) == 0ull) break;
          if (++spins > spin_limit) {
            // give up: report it through *nnz, then go on with what is there so that
            // the grid drains (offsets stay below n, the output is garbage)
            if (lane == 0) {
              atomicOr(&ws[1], 1u);
              atomicMin(nnz, -1);
              __threadfence();
            }
#pragma unroll
            for (int r = 0; r < 4; r++) v[r] |= kFlagPre;
            break;
          }
          __builtin_amdgcn_s_sleep(1);
        }
#pragma unroll
        for (int r = 0; r < 4; r++) {
          if (!done) {
            const unsigned long long pre = __ballot((v[r] >> 30) == 2u);
            unsigned take = 64;  // lanes 0..take-1 of this row contribute
            if (pre) { take = (unsigned)__builtin_ctzll(pre) + 1u; done = true; }
            unsigned contrib = lane < take ? (v[r] & kValMask) : 0u;
            excl += (unsigned)wave_sum((int)contrib);
          }
        }
        idx -= 256;
      }
      if (lane == 0) st_status(&status[tile], kFlagPre | ((excl + tile_agg) & kValMask));
    }
    if (lane == 0) s_tile = excl;
  }
  __syncthreads();
  unsigned off = s_tile;
#pragma unroll
  for (int w = 0; w < WAVES; w++) off += w < wv ? s_agg[w] : 0u;

  if (!in_layout) return;
  uint32_t* mrow = mask + (size_t)c * g.W;
  if (!has_data) {  // chunk without data: the reference leaves these words untouched; define them
    for (int w = lane; w < g.W; w += 64) mrow[w] = 0;
    return;
  }
  if (lane == 0) {
    begin[c] = (int)off;
    if (c == g.active - 1) atomicMin(nnz, (int)(off + agg));
  }

  // ---- phase 2: mask words and packed values from the registers
  uint32_t held = 0;
#pragma unroll
  for (int t = 0; t < IT; t++) {
    if (t < iters) {
      const bool nz = x[t] != 0.0f;
      const unsigned long long m = __ballot(nz);
      if (nz) values[off + rank_below(m)] = x[t];
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
  const size_t before = (size_t)g_staged_compact_bytes;
  g_staged_compact_bytes = bytes;
  return before;
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
  if (g.E % 4 == 0 && (reinterpret_cast<uintptr_t>(d_out) & 15u) == 0)
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

extern "C" size_t cswap_zvc_workspace_bytes(int process)
{
  return process > 0 ? ((size_t)process + 16) * sizeof(uint32_t) : 0;
}

extern "C" void cswap_zvc_debug_set_lookback(unsigned spin_limit, unsigned first_ticket)
{
  g_spin_limit = spin_limit ? spin_limit : kSpinLimit;
  g_first_ticket = first_ticket;
}

extern "C" int cswap_zvc_compress_fused(const float* d_in, int n, int process, void* d_ws, int* d_begin,
                                        int* d_nnz, float* d_values, uint32_t* d_mask, cswap_stream_t stream)
{
  if (!d_in || !d_ws || !d_begin || !d_nnz || !d_values || !d_mask) return CSWAP_E_ARG;
  Geometry g;
  int rc = make_geometry(g, n, process);
  if (rc) return rc;
  // chunks that do not fit a wavefront's registers, or prefixes that do not fit
  // the 30-bit status value, take the three-kernel path
  if (g.E > 64 * 128 || n >= (1 << 30)) return cswap_zvc_compress(d_in, n, process, d_begin, d_nnz, d_values, d_mask, stream);
  uint32_t* ws = (uint32_t*)d_ws;
  const int words = process + 16;
  hipLaunchKernelGGL(zvc_ws_zero_kernel, dim3((words + 255) / 256), dim3(256), 0, (hipStream_t)stream, ws, words,
                     (uint32_t)g_first_ticket, d_nnz);
  const int iters = (g.E + 63) >> 6;
#define CSWAP_FUSED(IT_, WAVES_)                                                                          \
  hipLaunchKernelGGL((zvc_fused_kernel<IT_, WAVES_>), dim3((g.process + WAVES_ - 1) / WAVES_),            \
                     dim3(64 * WAVES_), 0, (hipStream_t)stream, d_in, g, ws, d_begin, d_nnz, d_values, d_mask,   \
                     g_spin_limit)
  if (iters <= 8) CSWAP_FUSED(8, 16);
  else if (iters <= 16) CSWAP_FUSED(16, 16);
  else if (iters <= 32) CSWAP_FUSED(32, 16);
  else if (iters <= 64) CSWAP_FUSED(64, 8);
  else CSWAP_FUSED(128, 8);
#undef CSWAP_FUSED
  return check_launch();
}

// ------------------------------------------------------------------ no allocation
// The single-pass compression once more, for callers that cannot bring a workspace
// because they cannot allocate one: the status words live in this array, one copy
// per GPU, held until the process ends.
constexpr int kStaticProcessMax = 65536;
static __device__ __align__(256) uint32_t scratch[kStaticProcessMax + 16];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
uint32_t* g_scratch_ptr[kMaxDevices];  // device address of `scratch` on each GPU, once looked up
}  // namespace

extern "C" int cswap_zvc_compress_fused_static(const float* d_in, int n, int process, int* d_begin, int* d_nnz,
                                               float* d_values, uint32_t* d_mask, cswap_stream_t stream)
{
  if (process > kStaticProcessMax) return CSWAP_E_NOMEM;
  int dev = -1;
  CSWAP_HIP_TRY(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDevices) return CSWAP_E_UNSUPPORTED;
  uint32_t* ws;
  {
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {  // first call on this GPU: where its copy of the array lives
      void* p = nullptr;
      CSWAP_HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
      g_scratch_ptr[dev] = static_cast<uint32_t*>(p);
    }
    ws = g_scratch_ptr[dev];
  }
  return cswap_zvc_compress_fused(d_in, n, process, ws, d_begin, d_nnz, d_values, d_mask, stream);
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
