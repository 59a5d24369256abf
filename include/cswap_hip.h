/*
 * cswap_hip.h -- C ABI of libcswap_hip.so, the MI355X (gfx950) implementation of
 * the compression path CSWAP+ puts in front of GPU<->CPU activation swapping.
 *
 * Every pointer named d_* is device memory, h_* is host memory.  Every call
 * that launches work takes the HIP stream to launch on (a hipStream_t passed
 * as void*; NULL = the default stream) and returns without synchronising.
 * Return value: CSWAP_OK (0) or a negative CSWAP_E_* code; nothing throws and
 * nothing is printed.  No entry point allocates device memory unless its
 * comment says so.
 *
 * Each declaration cites the reference interface it stands in for
 * (paths relative to the reference tree, CSWAP+/...).
 */
#ifndef CSWAP_HIP_H
#define CSWAP_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define CSWAP_OK            0
#define CSWAP_E_ARG        -1  /* null pointer, zero size, size out of range */
#define CSWAP_E_UNSUPPORTED -2 /* valid request this build does not implement */
#define CSWAP_E_HIP        -3  /* a HIP runtime call failed (see cswap_last_hip_error) */
#define CSWAP_E_NOMEM      -4  /* pool or caller-provided buffer too small */
#define CSWAP_E_STATE      -5  /* call out of order (e.g. swap-in before swap-out) */

typedef void* cswap_stream_t; /* hipStream_t */

const char* cswap_strerror(int code);
int         cswap_last_hip_error(void); /* hipError_t of the last CSWAP_E_HIP on this thread */
int         cswap_abi_version(void);

/* ------------------------------------------------------------------ ZFP -----
 * Fixed-rate ZFP of a 3-D fp32 field a[nz][ny][nx] (x fastest).  Strides are in
 * elements; 0 means the contiguous default (sx=1, sy=nx, sz=nx*ny), as in
 * zfp/cuZFP.cu:372-375.  maxbits = bits per 4x4x4 block (64 * bits-per-value),
 * 16 <= maxbits <= 4096; block b owns stream bits [b*maxbits, (b+1)*maxbits)
 * (zfp/encode.cuh:229-230), blocks numbered x fastest (zfp/encode3.cuh:79-87).
 */

/* Stream size the reference reports: whole 64-bit words, rounded down
 * (zfp/encode3.cuh:147, zfp/shared.h:73-84). */
size_t cswap_zfp_stream_bytes(size_t nx, size_t ny, size_t nz, unsigned maxbits);
/* Bytes the stream buffer must hold: whole words, rounded up.  Equal to the
 * above whenever blocks*maxbits is a multiple of 64. */
size_t cswap_zfp_stream_capacity(size_t nx, size_t ny, size_t nz, unsigned maxbits);

/* Replaces cuZFP::encode<float> / encode3launch (zfp/encode3.cuh:117-199) as
 * reached from cuda_compress (zfp/cuZFP.cu:364-436).  Writes every word of the
 * stream (no prior memset needed). */
int cswap_zfp_compress_f32(const float* d_in, size_t nx, size_t ny, size_t nz,
                           ptrdiff_t sx, ptrdiff_t sy, ptrdiff_t sz, unsigned maxbits,
                           uint64_t* d_stream, cswap_stream_t stream);

/* Replaces cuZFP::decode3<float> (zfp/decode3.cuh:108-187) as reached from
 * cuda_decompress (zfp/cuZFP.cu:440-532).  Writes every element of the field. */
int cswap_zfp_decompress_f32(const uint64_t* d_stream, size_t nx, size_t ny, size_t nz,
                             ptrdiff_t sx, ptrdiff_t sy, ptrdiff_t sz, unsigned maxbits,
                             float* d_out, cswap_stream_t stream);

/* 1-D (4-value blocks) and 2-D (4x4 blocks) fields, as dispatched by
 * internal::encode / internal::decode on the number of non-zero dimensions
 * (zfp/cuZFP.cu:105-203; zfp/encode1.cuh, encode2.cuh, decode1.cuh, decode2.cuh).
 * dims = 1, 2 or 3; unused extents and strides are ignored; dims = 3 is the call
 * above.  maxbits is bits per block of 4^dims values.  For 1-D and 2-D the
 * reference reports the stream size rounded up to whole words (zfp/shared.h:42-71). */
size_t cswap_zfp_stream_capacity_nd(int dims, size_t nx, size_t ny, size_t nz, unsigned maxbits);
size_t cswap_zfp_stream_bytes_nd(int dims, size_t nx, size_t ny, size_t nz, unsigned maxbits);
int cswap_zfp_compress_f32_nd(const float* d_in, int dims, size_t nx, size_t ny, size_t nz,
                              ptrdiff_t sx, ptrdiff_t sy, ptrdiff_t sz, unsigned maxbits,
                              uint64_t* d_stream, cswap_stream_t stream);
int cswap_zfp_decompress_f32_nd(const uint64_t* d_stream, int dims, size_t nx, size_t ny, size_t nz,
                                ptrdiff_t sx, ptrdiff_t sy, ptrdiff_t sz, unsigned maxbits,
                                float* d_out, cswap_stream_t stream);
/* int32 fields (zfp_type_int32 in cuda_compress / cuda_decompress,
 * zfp/cuZFP.cu:412-416,513-517): the same transform and coder applied to the
 * values themselves -- no exponent header, no cast, the whole maxbits is the
 * coder's budget (zfp/encode.cuh:371-380,393-402,415-424).  Same stream sizes as
 * above. */
int cswap_zfp_compress_i32_nd(const int32_t* d_in, int dims, size_t nx, size_t ny, size_t nz,
                              ptrdiff_t sx, ptrdiff_t sy, ptrdiff_t sz, unsigned maxbits,
                              uint64_t* d_stream, cswap_stream_t stream);
int cswap_zfp_decompress_i32_nd(const uint64_t* d_stream, int dims, size_t nx, size_t ny, size_t nz,
                                ptrdiff_t sx, ptrdiff_t sy, ptrdiff_t sz, unsigned maxbits,
                                int32_t* d_out, cswap_stream_t stream);
/* double and int64 fields (zfp_type_double, zfp_type_int64 in cuda_compress /
 * cuda_decompress, zfp/cuZFP.cu:401-411,418-423,479-504): 64 bit planes over
 * int64 coefficients; doubles carry a 12-bit block header (flag + 11-bit
 * exponent, zfp/type_info.cuh:8-17) and are scaled by 2^(62-emax)
 * (zfp/encode.cuh:136-149); int64 has no header.  Strides are in elements;
 * d_in / d_out must be 8-byte aligned.  maxbits counts bits per block of 4^dims
 * values as above (so a rate of r bits per value is maxbits = r * 4^dims). */
int cswap_zfp_compress_f64_nd(const double* d_in, int dims, size_t nx, size_t ny, size_t nz,
                              ptrdiff_t sx, ptrdiff_t sy, ptrdiff_t sz, unsigned maxbits,
                              uint64_t* d_stream, cswap_stream_t stream);
int cswap_zfp_decompress_f64_nd(const uint64_t* d_stream, int dims, size_t nx, size_t ny, size_t nz,
                                ptrdiff_t sx, ptrdiff_t sy, ptrdiff_t sz, unsigned maxbits,
                                double* d_out, cswap_stream_t stream);
int cswap_zfp_compress_i64_nd(const int64_t* d_in, int dims, size_t nx, size_t ny, size_t nz,
                              ptrdiff_t sx, ptrdiff_t sy, ptrdiff_t sz, unsigned maxbits,
                              uint64_t* d_stream, cswap_stream_t stream);
int cswap_zfp_decompress_i64_nd(const uint64_t* d_stream, int dims, size_t nx, size_t ny, size_t nz,
                                ptrdiff_t sx, ptrdiff_t sy, ptrdiff_t sz, unsigned maxbits,
                                int64_t* d_out, cswap_stream_t stream);

/* No counterpart in the reference (which launches one thread per block whatever the
 * field's size, encode3.cuh:149-151, decode3.cuh:139-141).  A field of fewer than about
 * a million blocks does not fill this GPU with one lane per block; below these sizes in
 * bytes (of the uncompressed fp32 field) the 3-D fp32 kernels run in their pair form
 * instead -- two wavefronts share 64 blocks, each doing half of every phase -- where the
 * shape allows it: extents that are multiples of 4, contiguous 16-byte aligned rows, a
 * 16-byte aligned stream, maxbits a multiple of 256.  Same stream, same values.
 * Below the limit the form is taken while all of the field's workgroups fit on the chip
 * at once (their LDS decides how many do: about 37 MB at 8 bits per value, 30 MB at 16,
 * 21 MB at 32), and by the decoder only from 16 bits per value on (at 8 it measured no
 * gain).  0 = never; SIZE_MAX = whenever the shape allows, whatever the size and rate
 * (tests and measurements).  Defaults: 40 MiB both.  `previous`, if not NULL, receives
 * the two values that were in force.  Process-wide. */
void cswap_zfp_set_pair_bytes(size_t encode_below, size_t decode_below, size_t* previous);

/* ------------------------------------------------------------------ ZVC -----
 * Zero-value compaction in the reference's format (zfp/compression.cu).  The
 * tensor of n fp32 elements is cut into `process` chunks of
 * E = ceil(n/process) elements (the reference uses process = 512*32,
 * Execution.h:50-52); chunk i owns W = ceil(E/32) mask words starting at word
 * i*W, bit k%32 of word k/32 set iff element E*i+k != 0, and its non-zeros
 * start at d_values[d_begin[i]].  0 < n < 2^31, 0 < process <= 2^20.
 */
int    cswap_zvc_chunk_elems(int n, int process);   /* E */
int    cswap_zvc_chunk_words(int n, int process);   /* W */
int    cswap_zvc_active_chunks(int n, int process); /* chunks that hold data = ceil(n/E) */
size_t cswap_zvc_mask_bytes(int n, int process);    /* W*process*4, Execution.h:88 */
/* A good chunk count for n elements when the caller may choose (the reference
 * always passes 512*32): about 1024 elements per chunk, a power of two in
 * [1024, 16384].  Both directions must use the same value. */
int    cswap_zvc_pick_process(size_t n);
/* No counterpart in the reference: cswap_zvc_compact has two forms, one that
 * stores each 64-element row's non-zeros straight from the lanes that hold them
 * and one that stages them in LDS and writes whole aligned 1 KB runs with the
 * nontemporal hint; the second is faster for tensors larger than the GPU's
 * memory-side cache and runs for tensors of at least this many bytes (default
 * 192 MiB; 0 = always, SIZE_MAX = never).  Same output either way.  Returns the
 * previous value.  Process-wide; not meant to be changed while kernels are being launched. */
size_t cswap_zvc_set_staged_compact_bytes(size_t bytes);

/* Replaces PreGPUcompression (zfp/compression.cu:134-165, launcher :334-341):
 * d_count[i] = number of elements != 0 in chunk i, for the active chunks. */
int cswap_zvc_count(const float* d_in, int n, int process, int* d_count, cswap_stream_t stream);

/* Replaces PreAcc (zfp/compression.cu:9-19, launcher :342-350): in-place
 * exclusive prefix sum over the first k entries; *d_nnz = total. */
int cswap_zvc_scan(int* d_count, int k, int* d_nnz, cswap_stream_t stream);

/* Replaces GPUcompression (zfp/compression.cu:168-239, launcher :351-365).
 * d_values must hold nnz floats, d_mask cswap_zvc_mask_bytes(n,process).  Every
 * mask word is written (words the reference leaves untouched are zeroed). */
int cswap_zvc_compact(const float* d_in, int n, int process, const int* d_begin,
                      float* d_values, uint32_t* d_mask, cswap_stream_t stream);

/* Replaces GPUdecompression (zfp/compression.cu:241-318, launcher :367-374).
 * Unlike the reference it writes all n outputs (zeros as +0.0) and needs no
 * pre-zeroed destination. */
int cswap_zvc_expand(const float* d_values, const uint32_t* d_mask, const int* d_begin,
                     int n, int process, float* d_out, cswap_stream_t stream);

/* count + scan + compact in one call with no host round trip (the reference
 * copies nnz to the host between the steps, Execution.h:89-95).  d_values must
 * hold n floats (worst case); *d_nnz receives the total. */
int cswap_zvc_compress(const float* d_in, int n, int process, int* d_begin, int* d_nnz,
                       float* d_values, uint32_t* d_mask, cswap_stream_t stream);

/* The same result in a single pass over the tensor: resident workgroups walk the
 * tensor tile by tile, keep the tiles they have loaded in registers until a
 * scanner workgroup has turned the published tile counts into offsets, and then
 * write mask, offsets and packed values, so HBM traffic is the algorithmic
 * 4 + 1/8 + 4*density bytes per element.  Smaller tensors than
 * cswap_zvc_set_single_pass_bytes says (64 MiB) do not fill that pipeline; of those,
 * tensors whose mask layout has at most 131072 rows of 64 elements (32 MiB) run
 * another one-kernel form -- the whole tensor in the registers of one grid, every
 * workgroup reads the counts of the workgroups before it -- and the rest the three kernels.  d_ws is a
 * workspace of cswap_zvc_workspace_bytes(process) bytes (at least 256 KiB) that
 * cswap_zvc_workspace_clear has prepared once, after it was allocated; every call
 * that succeeds leaves it ready for the next one (the kernel clears each status
 * word as it consumes it, so no launch is spent on clearing); calls that share a
 * workspace must not overlap.  Shapes the one-kernel forms do not take -- a chunk
 * length that is not a multiple of 32, for the pipeline d_values not 16-byte
 * aligned or more than 32512 tiles of 12288 elements -- run the three kernels instead.  The workgroups
 * wait for each other's counts; that wait is bounded, and if it ever runs out (for
 * example because the pipeline kernel, whose 256 workgroups all have to run at the
 * same time, does not get the whole GPU) the kernel still finishes
 * but *d_nnz is -1 and the other outputs are undefined: a caller must treat a
 * negative count as failure (the return value cannot tell, the call does not
 * synchronise).  A workspace that was never prepared is reported the same way, and
 * so is every later call on a workspace after a failure, until
 * cswap_zvc_workspace_clear has been called on it again. */
size_t cswap_zvc_workspace_bytes(int process);
int cswap_zvc_compress_fused(const float* d_in, int n, int process, void* d_ws, int* d_begin,
                             int* d_nnz, float* d_values, uint32_t* d_mask, cswap_stream_t stream);
/* No counterpart in the reference.  Prepares a workspace of
 * cswap_zvc_workspace_bytes(process) bytes for cswap_zvc_compress_fused (one small
 * kernel on `stream`): once after allocating it, and again after a call that
 * reported failure.  d_ws == NULL: the static workspace of
 * cswap_zvc_compress_fused_static on the current GPU (which starts out prepared;
 * `process` is ignored). */
int cswap_zvc_workspace_clear(void* d_ws, int process, cswap_stream_t stream);
/* What cswap_zvc_compress_fused would run for this shape (given a 16-byte aligned
 * d_values): 1 the pipeline kernel, 2 the one-kernel form for small tensors, 0 the
 * three kernels.  Host only. */
int cswap_zvc_takes_single_pass(int n, int process);
/* No counterpart in the reference: the tensor size in bytes from which
 * cswap_zvc_compress_fused runs the pipeline kernel (default 64 MiB; 0 = whenever
 * the shape allows, and then the form for small tensors never runs; SIZE_MAX =
 * the three kernels for every tensor).
 * Returns the previous value.  Process-wide. */
size_t cswap_zvc_set_single_pass_bytes(size_t bytes);
/* No counterpart in the reference.  cswap_zvc_compress_fused for callers that
 * cannot allocate a workspace (code under HIP graph capture, serving loops and
 * harnesses that forbid hipMalloc): the status words live in a static device
 * array of the library (256 KiB per GPU, held until the process ends), so the
 * call takes no workspace and allocates nothing.  process <= 65536, otherwise
 * CSWAP_E_NOMEM.  Every call on a GPU uses that GPU's one array: calls that
 * overlap on one GPU (different streams, different threads) race.  After a call
 * that reported failure (*d_nnz == -1), cswap_zvc_workspace_clear(NULL, 0, stream)
 * makes the array usable again. */
int cswap_zvc_compress_fused_static(const float* d_in, int n, int process, int* d_begin, int* d_nnz,
                                    float* d_values, uint32_t* d_mask, cswap_stream_t stream);

/* ---------------------------------------------------------------- probe -----
 * One fused read pass: *d_nnz = number of elements != 0 (the quantity the
 * reference derives from PreGPUcompression + PreAcc, Execution.h:89-92). */
int cswap_probe_nnz(const float* d_in, size_t n, unsigned long long* d_nnz, cswap_stream_t stream);

/* -------------------------------------------------------------- selector -----
 * Per-tensor choice between no compression, ZVC and fixed-rate ZFP.  The
 * reference's selector (c10::GetPolicyMaker()->make_policy, call sites
 * cp-vgg16.cpp:513 and vgg16-cifar10.cpp:481) is not in its tree; README.md:6
 * describes it as weighing compression ratio, size and algorithm
 * characteristics at run time.  This one minimises a modelled swap-out +
 * swap-in latency:  t(option) = t_compress + bytes_out/bw_d2h + bytes_out/bw_h2d
 * + t_decompress (+ fixed per-kernel and per-copy overheads, + the cost of the
 * probe itself for the compressed options), with kernel times
 * = bytes_in / throughput; a compressed option is taken only if it is modelled
 * faster than min_gain * the raw swap.  Ties go to the lossless option; ZVC is only
 * eligible when its size ratio is below sparse_max_ratio; tensors below
 * size_floor_bytes are never compressed.  Lossless is preferred: when ZVC beats
 * the raw swap, lossy ZFP replaces it only if it is modelled at least
 * 1/lossy_min_gain times faster (the reference's hand-written policies give ZVC
 * to ReLU outputs and ZFP to dense/pooled tensors, vgg16-cifar10.cpp:177-178,
 * 393-397).
 */
typedef enum { CSWAP_POLICY_AUTO = -1, CSWAP_POLICY_NONE = 2, CSWAP_POLICY_SPARSE = 3,
               CSWAP_POLICY_ZFP = 6, /* codes as in Execution.h:70,86,107 */
               /* The selector again, for a tensor that is expected to be sparse (the caller
                * remembers that the selector chose ZVC for it the last time): the engine runs the
                * ZVC compaction right away, in its single-kernel form, which produces the count on
                * the way -- the reference's one probe is likewise the count pass of its compactor
                * (Execution.h:89-95) -- and asks the selector with that count.  If the answer is
                * still ZVC the payload is there already; if not, the selector's choice runs as
                * it would have after a probe.  Never a wrong result, one wasted pass when the
                * expectation was wrong. */
               CSWAP_POLICY_AUTO_SPARSE = -3 } cswap_policy;

typedef struct {
  double bw_d2h_gbs, bw_h2d_gbs;         /* pinned host link, GB/s */
  double copy_latency_us;                /* fixed cost of one async copy */
  double kernel_latency_us;              /* fixed cost of one ZVC kernel */
  double zfp_latency_us;                 /* fixed cost of one ZFP kernel: a lone wavefront's serial work, which a
                                            tensor too small to fill the chip cannot go below */
  double zvc_compress_gbs, zvc_expand_gbs; /* GB/s of fp32 in / out */
  double zfp_compress_gbs, zfp_decompress_gbs;
  double sparse_max_ratio;               /* ZVC eligible only below this size ratio */
  double lossy_min_gain;                 /* ZFP replaces a winning ZVC only if t_zfp < gain * t_zvc */
  double probe_latency_us;               /* fixed cost of deciding: counting kernels + host round trip */
  double probe_gbs;                      /* throughput of the counting pass, GB/s of fp32 in */
  double min_gain;                       /* compress only if modelled time < min_gain * raw swap time */
  int    d2h_hidden;                     /* 1: assume the outbound copy overlaps compute (only the
                                            inbound copy, kernels and probe are on the critical path) */
  size_t size_floor_bytes;               /* never compress smaller tensors */
  int    allow_lossy;                    /* 0: ZFP is never chosen */
  int    process;                        /* ZVC chunk count (512*32 in the reference) */
} cswap_costs;

typedef struct {
  int    policy;            /* CSWAP_POLICY_NONE / SPARSE / ZFP */
  size_t bytes_out;         /* bytes that cross the host link, one way */
  double ratio;             /* bytes_out / (4*n) */
  double t_none_us, t_sparse_us, t_zfp_us; /* modelled swap-out + swap-in latency */
} cswap_choice;

/* Defaults measured on one MI355X box (see cswap_calibrate to re-measure). */
void cswap_costs_default(cswap_costs* c);
/* Bytes a tensor of n elements with nnz non-zeros occupies under each policy. */
size_t cswap_policy_bytes(int policy, size_t n, size_t nnz, unsigned maxbits, int process,
                          size_t nx, size_t ny, size_t nz);
/* Pure host functions, no GPU work.  cswap_select sees a flat tensor (ZFP size
 * = ceil(n/64) blocks); cswap_select_field uses the true block count of the
 * field a[nz][ny][nx], which matters when nx or ny is not a multiple of 4
 * (a 2x2xN field pays the full rate for blocks that are 3/4 padding). */
int cswap_select(size_t n, size_t nnz, unsigned maxbits, const cswap_costs* costs, cswap_choice* out);
int cswap_select_field(size_t nx, size_t ny, size_t nz, size_t nnz, unsigned maxbits,
                       const cswap_costs* costs, cswap_choice* out);

/* ----------------------------------------------------------- swap engine -----
 * Mirror of Execution::init_/pre/post (Execution.h:46-133,217-310) and of the
 * backward-side swap-in the reference keeps in its patched autograd
 * (com_and_tran tags, Execution.h:262,280,299).  One engine owns a copy stream
 * (default priority, non-blocking), a pinned host pool and a device staging
 * pool, all allocated once in cswap_engine_create and freed in
 * cswap_engine_destroy; the swap calls themselves do not allocate.
 */
typedef struct cswap_engine cswap_engine;

typedef struct {
  size_t pinned_pool_bytes;   /* host side: compressed tensors live here while swapped out */
  size_t device_pool_bytes;   /* device staging for compressed data in flight: every tensor between swap_out and
                                 the end of its outbound copy, and between prefetch / swap_in and the end of its
                                 decompression, holds a block of its compressed size (raw swaps hold none going
                                 out).  Blocks come back as that work finishes, without anybody waiting; a
                                 request that finds the pool full waits for the oldest work in flight, and only
                                 when nothing in flight can make room does an AUTO request go out raw and an
                                 explicit one return CSWAP_E_NOMEM (a prefetch, being optional, waits only for
                                 what released tickets still hold). */
  int    process;             /* ZVC chunk count; 0 = per tensor size (cswap_engine_tune result, else cswap_zvc_pick_process) */
  unsigned zfp_maxbits;       /* bits per 4x4x4 block for policy ZFP; 0 = 512 (8 bits/value) */
  int    max_tickets;         /* tensors that may be swapped out at once; 0 = 256 */
  cswap_costs costs;          /* used by CSWAP_POLICY_AUTO; zero bw fields = defaults */
  int    timing;              /* not 0: every phase of a ticket is bracketed by timing events on the stream it
                                 runs on and cswap_swap_timing reports them (the reference's profiler slots,
                                 Execution.h:109-126,285-295).  0 (default): events carry no timestamps. */
} cswap_engine_config;

typedef struct {
  int    policy;              /* what was actually done */
  size_t n, nnz;              /* elements; non-zeros (valid when probed) */
  size_t bytes_in, bytes_out; /* 4*n; bytes that crossed the link */
  int    state;               /* 0 free, 1 out in flight, 2 resident on host, 3 in in flight, 4 prefetched */
} cswap_ticket_info;

/* What a ticket's phases took on the GPU, in microseconds, from events recorded on the stream
 * each phase runs on (engines created with config.timing only).  -1: that phase has not
 * finished yet (or never started); 0: it did not take place (a raw swap has no kernels; a
 * tensor that came back from its staging block crossed the link only once).
 *   compress_us    from the call of cswap_swap_out on the compute stream to the end of the
 *                  compression kernel: probe or single-pass count, the host round trip for
 *                  the count, the selector, the compression (the reference's slot 2,
 *                  Execution.h:109-116, which also starts before `compress` and ends after it)
 *   copy_out_us    the device-to-host copy on the copy stream (what the reference splits into
 *                  the part under the consumer's kernel, slot 0, and the wait after it,
 *                  slot 1: Execution.h:285-295)
 *   copy_in_us     the host-to-device copy on the inbound copy stream
 *   decompress_us  the decompression kernel on the compute stream */
typedef struct {
  double compress_us, copy_out_us, copy_in_us, decompress_us;
} cswap_ticket_timing;

void cswap_engine_config_default(cswap_engine_config* cfg);
int  cswap_engine_create(cswap_engine** out, const cswap_engine_config* cfg);
void cswap_engine_destroy(cswap_engine* e);

/* Execution::pre: compress d_in on `compute` (policy AUTO probes and selects
 * first, which costs one small host round trip like Execution.h:92) and start
 * the device-to-host copy on the engine's copy stream, ordered after the
 * compression by an event.  The tensor is the field a[nz][ny][nx].
 * The probe of an AUTO request is the counting pass of the compactor, whose per-chunk
 * counts the compaction then reuses (Execution.h:89-95); for tensors small enough for the
 * one-kernel form of the compactor (cswap_zvc_takes_single_pass == 2, up to 32 MiB) it is
 * that kernel itself, into a staging block of the worst-case size when the pool has one
 * to spare: a tensor that turns out sparse is compacted by the time its count is known.
 * Calls that probe hold the engine's lock over the host round trip (about 20 us): two
 * threads' swap-outs through one engine take turns. */
int cswap_swap_out(cswap_engine* e, const float* d_in, size_t nx, size_t ny, size_t nz, int policy,
                   cswap_stream_t compute, int* ticket);
/* Execution::post: block the host until the copy of `ticket` has finished;
 * afterwards the caller may free or overwrite the device tensor.  Required for a
 * raw swap only (policy NONE in cswap_swap_info), whose copy reads the tensor
 * itself: a compressed swap has read it on `compute` by the time cswap_swap_out
 * returns, so it may go back to a stream-ordered allocator at once and nobody
 * has to wait.  Also answered after a cswap_swap_in that came first. */
int cswap_swap_wait(cswap_engine* e, int ticket);
/* Backward side: copy back on the engine's inbound copy stream (its own: both
 * directions of the link can be busy at once), then decompress into d_out on
 * `compute` (ordered by an event).  Returns at once; the data is ready when
 * `compute` reaches this point.  A compressed tensor whose outbound copy has not
 * finished yet is still in its staging block and is decompressed from there: no
 * wait for the copy, nothing on the link. */
int cswap_swap_in(cswap_engine* e, int ticket, float* d_out, cswap_stream_t compute);
/* Backward side, ahead of time: start the host-to-device copy of the payload
 * into the engine's device staging pool on the copy stream, before a
 * destination exists, so that it overlaps the backward compute of the layers
 * that run first.  A later cswap_swap_in then only waits for that copy and
 * decompresses (policy NONE: one device-to-device copy).  For a compressed tensor
 * whose outbound copy is still in flight the payload is on the device already: it
 * is kept there and nothing is copied.  Idempotent; the
 * reference's counterpart lives in its patched autograd engine, which it does
 * not ship (fields read at Execution.h:260-262,278-282). */
int cswap_swap_prefetch(cswap_engine* e, int ticket);
/* Give the ticket up.  Returns at once: its host (and any device) memory goes back
 * to the pools when the work of the ticket that is still in flight has finished,
 * and the ticket number is not handed out again before that. */
int cswap_swap_release(cswap_engine* e, int ticket);
int cswap_swap_info(cswap_engine* e, int ticket, cswap_ticket_info* info);
/* Phase times of a ticket so far (see cswap_ticket_timing); does not wait for anything.
 * CSWAP_E_UNSUPPORTED on an engine created without config.timing. */
int cswap_swap_timing(cswap_engine* e, int ticket, cswap_ticket_timing* out);
/* The ZFP rate (bits per 4x4x4 block, 16..4096) of the swap-outs from now on;
 * config.zfp_maxbits until it is called.  Replaces setRatio(int) called from the
 * training loop (CSWAP+/Execution.h:63; CIFAR10/cifar10.py:106 sets it every
 * epoch): maxbits = 4 * ratio.  A ticket keeps the rate it was swapped out with,
 * so tensors that are on the host or in flight come back correctly whatever is
 * set in between.  (The cost model's ZFP throughput figures stay those of the
 * rate the engine was calibrated with.) */
int cswap_engine_set_zfp_maxbits(cswap_engine* e, unsigned maxbits);
/* Number of probes so far: counting passes followed by the host round trip for
 * the non-zero count (the one at Execution.h:92), which a selector-driven or ZVC
 * swap-out pays and an explicit raw or ZFP request does not. */
unsigned long long cswap_engine_probe_count(cswap_engine* e);
/* Measure link bandwidth and kernel throughput on this box and store them in
 * the engine's cost model (allocates temporaries; call once after create). */
int cswap_engine_calibrate(cswap_engine* e, cswap_costs* out_costs);
/* Launch-geometry self-tuning.  The reference hands dimsize x blocksize (the
 * chunk count) to every ZVC entry point and always uses 512 x 32
 * (zfp/compression.cu:334-374).  With config.process == 0 the engine picks the
 * chunk count per tensor: cswap_engine_tune(e, n, &best) times count + scan +
 * compact + expand for power-of-two chunk counts on a synthetic tensor of n
 * elements (allocates temporaries) and remembers the winner for tensors of that
 * size class (same bit length of n); sizes never tuned use
 * cswap_zvc_pick_process.  cswap_engine_process_for reports the chunk count the
 * engine would use for a tensor of n elements. */
int cswap_engine_tune(cswap_engine* e, size_t n, int* best_process);
int cswap_engine_process_for(cswap_engine* e, size_t n);
cswap_stream_t cswap_engine_copy_stream(cswap_engine* e);

/* --------------------------------------------------------------- planner -----
 * Which activations to move off the device, and with which action, so that a
 * given share of the activation bytes leaves the device at the least predicted
 * cost.  Stands in for c10::PolicyMaker of the reference's patched PyTorch
 * (definitions not in its tree; driven as at inception-v3-cifar100.cpp:207-214
 * and vgg16-cifar10.cpp:474-497).  Pure host code.  Tensor id = index of the op
 * that produced it; ops are numbered in the order of cswap_planner_add_comptime.
 */
typedef struct cswap_planner cswap_planner;

typedef struct {
  double time_us;        /* predicted iteration time with the plan */
  double base_time_us;   /* predicted iteration time with nothing swapped */
  size_t bytes_total;    /* bytes of all recorded tensors */
  size_t bytes_target;   /* ratio * bytes_total */
  size_t bytes_moved;    /* device bytes the plan moves to the host */
  size_t bytes_on_link;  /* bytes that cross the link one way under the plan */
  int    n_selected;
  int    target_met;     /* 0: every eligible tensor is selected and it is still not enough */
} cswap_plan_summary;

/* costs NULL (or without link bandwidth) = cswap_costs_default; zfp_maxbits 0 = 512 */
cswap_planner* cswap_planner_create(const cswap_costs* costs, unsigned zfp_maxbits);
void cswap_planner_destroy(cswap_planner* p);
int  cswap_planner_reset(cswap_planner* p);
/* backward time of an op = factor * its forward time (default 2) */
int  cswap_planner_set_backward_factor(cswap_planner* p, double factor);
/* PolicyMaker::add_comptime(timeuse): forward time of the next op */
int  cswap_planner_add_comptime(cswap_planner* p, double microseconds);
/* PolicyMaker::add_tensor(index, x.nbytes()) */
int  cswap_planner_add_tensor(cswap_planner* p, int id, size_t nbytes);
/* PolicyMaker::add_stepdep({pre.tensor_id, index}): op to_id consumes tensor from_id (-1: untracked input) */
int  cswap_planner_add_stepdep(cswap_planner* p, int from_id, int to_id);
/* PolicyMaker::add_omitid(id): never touch this tensor */
int  cswap_planner_add_omitid(cswap_planner* p, int id);
/* What the reference's profile cannot know: the field extents (exact ZFP size)
 * and the non-zero count of the profiled iteration (enables ZVC for the tensor). */
int  cswap_planner_set_field(cswap_planner* p, int id, size_t nx, size_t ny, size_t nz);
int  cswap_planner_set_nnz(cswap_planner* p, int id, size_t nnz);
/* PolicyMaker::init(ratio): share of the recorded bytes to move off the device, 0..1 */
int  cswap_planner_init(cswap_planner* p, double ratio);
/* PolicyMaker::make_policy(time_): policy[id] in {0 keep, 2 raw, 3 ZVC, 6 ZFP}
 * (Execution.h:70,86,107) and begin_stage[id] = op of the last forward use
 * (what read_lastvisit fills, resnet-cifar10.cpp:330); both arrays have n entries,
 * begin_stage may be NULL. */
int  cswap_planner_make_policy(cswap_planner* p, int* policy, int* begin_stage, int n, cswap_plan_summary* summary);
/* PolicyMaker::capuchin(time_): the raw-swap baseline (action 2 only, tensors
 * that stay away longest first). */
int  cswap_planner_capuchin(cswap_planner* p, int* policy, int* begin_stage, int n, cswap_plan_summary* summary);

#ifdef __cplusplus
}
#endif
#endif /* CSWAP_HIP_H */
