/*
 * vtkv - C ABI of the MI355X (gfx950) vTensor KV-cache hot path.
 *
 * Every entry point takes plain pointers and sizes (no framework types), returns
 * 0 on success or a negative VTKV_E* code, and leaves a human-readable message in
 * vtkv_last_error().  Device pointers are HIP device addresses of the current
 * device; `stream` is a hipStream_t passed as void* (NULL = the null stream).
 * All kernels are asynchronous on `stream`; nothing here synchronises unless the
 * comment says so.
 *
 * Each declaration cites the interface of the reference (paths relative to its
 * GLakeServe/ directory) that it replaces.
 */
#ifndef VTKV_H
#define VTKV_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif
/* the library is built with hidden visibility: what is declared here is what it exports */
#pragma GCC visibility push(default)

#define VTKV_OK 0
#define VTKV_EINVAL (-1)   /* bad argument (shape, dtype, alignment, null pointer)      */
#define VTKV_EHIP (-2)     /* a HIP runtime call failed                                 */
#define VTKV_ENOMEM (-3)   /* physical chunk pool exhausted / workspace too small       */
#define VTKV_ESTATE (-4)   /* call order violated (pool not initialised, double free …) */

/* element types */
#define VTKV_F32 0
#define VTKV_BF16 1
#define VTKV_F16 2
#define VTKV_FP8_E4M3 3 /* OCP e4m3fn, one byte per element, per-tensor scale */

/* copy directions for vtkv_swap_* */
#define VTKV_D2H 0
#define VTKV_H2D 1
#define VTKV_D2D 2

/* Message of the last failing call on this thread ("" if none). */
const char *vtkv_last_error(void);
/* ABI version: major*10000 + minor*100 + patch. */
int vtkv_version(void);

/* ------------------------------------------------------------------------------------------
 * Physical chunk pool and per-sequence virtual ranges.
 * Replaces the pybind module `vmmAllocator` (vmm_allocator/vmm_allocator.h:190-219).
 * ---------------------------------------------------------------------------------------- */

/* Size of one physical chunk in bytes (2 MiB unless changed; vmm_allocator/vmm_allocator.h:45
 * granularitySize). */
int64_t vtkv_chunk_bytes(void);
/* Use chunks of `bytes` (a power of two from 2 MiB to 1 GiB) from the next vtkv_pool_init on.  Only while the
 * pool is empty: before the first vtkv_pool_init or after vtkv_pool_destroy (VTKV_ESTATE otherwise).  The
 * reference's granularity is fixed at 2 MiB; a pool holds at most 30000 chunks with this HIP runtime (see
 * vtkv_pool_init), so a cache above 58 GiB needs larger ones: 16 MiB chunks serve up to 468 GiB.  Every size
 * and offset the other calls take in chunks or require to be chunk multiples then refers to this size. */
int vtkv_pool_set_chunk_bytes(int64_t bytes);

/* Create `num_chunks` physical chunks on `device` and keep them in the free pool.
 * Replaces init_physical_handle(num_blocks, device_id) (vmm_allocator.cpp:113-151).
 * May be called again to add chunks.  At most 30000 chunks in all (VTKV_EINVAL beyond): the HIP runtime
 * has 65536 entries per process for physical chunks and their mappings together; larger caches take larger
 * chunks (vtkv_pool_set_chunk_bytes). */
int vtkv_pool_init(int device, int64_t num_chunks);
/* Chunks no sequence owns; replaces showFreeBlocks() (vmm_allocator.cpp:472-474). <0 on error.
 * Unmapping is lazy: a segment that shrinks (preempt, release, swap-out) keeps its chunks mapped at the
 * top of its ranges as "retired" chunks, which count as free here; they are unmapped when another
 * segment needs them, and taken back without a driver call if the same segment grows again first. */
int64_t vtkv_pool_free_chunks(void);
/* How many of the free chunks are retired, i.e. still mapped.  No counterpart in the reference. */
int64_t vtkv_pool_retired_chunks(void);
/* Physical chunks the pool has released and created anew so far: a chunk is replaced after 256 mappings,
 * or earlier once the live chunks of the pool have been through more mappings than its share of the
 * runtime's entries, because the HIP runtime keeps an entry for every address a chunk was ever mapped at
 * until the chunk is released, and runs out of them otherwise.  No counterpart in the reference. */
int64_t vtkv_pool_recreated_chunks(void);
/* Unmap retired chunks now, until at least `max_chunks` are unmapped or none is left (< 0: all; whole
 * rows, i.e. one chunk of every range of a segment, at a time), so that later growth finds them on the
 * free list; meant for idle moments of the host thread.  Returns the number unmapped, < 0 on error.
 * No counterpart in the reference (its release path unmaps at once, vmm_allocator.cpp:393-420). */
int64_t vtkv_pool_trim(int64_t max_chunks);
/* Chunks ever created and still owned (free + mapped). */
int64_t vtkv_pool_total_chunks(void);
/* Release every chunk and every segment's address range.  All segments must have been destroyed. */
int vtkv_pool_destroy(void);

typedef struct vtkv_segment vtkv_segment;

/* One sequence slot: for each of `layer_num` layers a K range and a V range of
 * `context_max_bytes` reserved virtual addresses; nothing mapped unless `expand` is non-zero, in
 * which case expand_bytes/chunk chunks are mapped at once.  `expand_bytes` is also what release
 * keeps mapped.  Replaces KVcacheSegment(layer_num, context_max_size, expand_size, expand)
 * (vmm_allocator.cpp:177-211).  Returns NULL on failure. */
vtkv_segment *vtkv_seg_create(int layer_num, int64_t context_max_bytes, int64_t expand_bytes, int expand);
/* Unmap everything, return the chunks to the pool and free the address ranges (the reference never frees them). */
int vtkv_seg_destroy(vtkv_segment *seg);
/* Base device address of the K / V range of `layer`; replaces getKeyDevicePtr / getValueDevicePtr
 * (vmm_allocator.cpp:299-305).  0 on error. */
uint64_t vtkv_seg_key_ptr(const vtkv_segment *seg, int layer);
uint64_t vtkv_seg_value_ptr(const vtkv_segment *seg, int layer);
/* Offset in bytes of the segment's V rows inside their V ranges (0 unless set): vtkv_seg_value_ptr and the V
 * pointer tables hand out range base + offset, the K rows start at the base.  The K and the V row of one
 * token and kv head are read together; in two chunk-aligned ranges they share every address bit below the
 * chunk size and meet in one memory channel, which costs 5 to 6 % of the streaming rate; 256 bytes apart they
 * do not.  Mapping counts the offset: the segment keeps used + offset <= mapped, so a range holds
 * (max bytes - offset) / row bytes rows and reaches a chunk boundary one row early; a caller that maps by
 * hand (vtkv_seg_expand) and writes through the pointers must count it too.  No counterpart in the reference,
 * which places both ranges at their base (vmm_allocator.cpp:177-212). */
int64_t vtkv_seg_value_skew(const vtkv_segment *seg);
/* Set that offset (a multiple of 256 up to 4096).  Only while the segment holds no rows (VTKV_ESTATE
 * otherwise); pointers and pointer-table entries fetched before the call are stale after it.  Both segments
 * of a vtkv_seg_share_prefix must use the same offset. */
int vtkv_seg_set_value_skew(vtkv_segment *seg, int64_t bytes);
/* used_size (bytes written per range) get/set; replaces get_used_slot / set_used_size (vmm_allocator.cpp:339-345). */
int64_t vtkv_seg_get_used(const vtkv_segment *seg);
int vtkv_seg_set_used(vtkv_segment *seg, int64_t used_bytes);
/* actual_size: bytes currently mapped per range (vmm_allocator.h:98). */
int64_t vtkv_seg_mapped_bytes(const vtkv_segment *seg);
/* Map `num_chunks` more chunks at the end of every K and V range of every layer (2*layers*num_chunks
 * chunks in total); replaces expandMultiSegment (vmm_allocator.cpp:214-297).  VTKV_ENOMEM leaves the
 * segment unchanged. */
int vtkv_seg_expand(vtkv_segment *seg, int num_chunks);
/* Prefill-side growth: make room for `token_bytes` more bytes plus a slack of 100*kv_size bytes, map the
 * chunks needed, then used += token_bytes.  Replaces KVcacheSegment::copy_kv_cache (vmm_allocator.cpp:322-337). */
int vtkv_seg_reserve(vtkv_segment *seg, int64_t token_bytes, int64_t kv_size);
/* Decode-side growth that the reference spreads over eagerExtend + its background thread
 * (vmm_allocator.cpp:40-72,307-320): map one more chunk when used + token_bytes would pass the mapped
 * size.  Returns 1 if a chunk was mapped, 0 if not, <0 on error. */
int vtkv_seg_ensure(vtkv_segment *seg, int64_t token_bytes);
/* Unmap all chunks, used = 0; replaces preempt_seq (vmm_allocator.cpp:348-381). */
int vtkv_seg_preempt(vtkv_segment *seg);
/* Unmap all but the first expand_bytes, used = 0; replaces release_seq (vmm_allocator.cpp:383-421). */
int vtkv_seg_release(vtkv_segment *seg);

/* Start `dst` (which must hold no rows) as a sequence that shares the first `bytes` bytes of every range
 * of `src`: whole chunks below that mark are mapped into dst's ranges as well (one physical chunk, two
 * addresses: no copy, no chunk taken from the pool), the partly filled chunk, if any, is copied into a
 * chunk of dst's own on `stream`, and dst's used size becomes `bytes`.  Both sequences only ever append
 * behind the prefix, so neither writes to a shared chunk.  A shared chunk returns to the pool when the
 * last segment that maps it gives it up.  Stands in for the prefix reuse that the reference's radix cache
 * plans but leaves unimplemented (vmm_allocator/radix_cache.py:184 `split_and_copy`). */
int vtkv_seg_share_prefix(vtkv_segment *dst, vtkv_segment *src, int64_t bytes, void *stream);
/* Physical chunks currently mapped into more than one segment.  No counterpart in the reference. */
int64_t vtkv_pool_shared_chunks(void);

/* Map `num_chunks` more chunks into every range of the segment on a worker thread and return at once;
 * replaces KVcacheSegment::eagerExtend and the eagerly_extend thread (vmm_allocator.cpp:40-72,307-320).
 * Nothing happens if the ranges are fully mapped.  Any later call that changes the segment, and
 * vtkv_extend_kv_cache_batch when a new row needs the chunk, first waits for the request.  A failed
 * request (pool exhausted) is reported once, by the next call that grows the segment (vtkv_seg_expand,
 * vtkv_seg_reserve, vtkv_seg_ensure, vtkv_seg_share_prefix as destination, vtkv_extend_kv_cache_batch);
 * calls that shrink it (vtkv_seg_preempt, vtkv_seg_release, vtkv_seg_destroy) forget the failure and do
 * their work, since a full pool is when a caller preempts to get chunks back.  The driver calls run
 * outside the pool's lock. */
int vtkv_seg_eager_extend(vtkv_segment *s, int num_chunks);
/* vtkv_seg_eager_extend(s, 1) for every segment of the list whose rows have come within `ahead_bytes` of the end
 * of what is mapped (used + ahead_bytes > mapped, the V offset counted), that has no request under way and that
 * the pool can serve at the time of the call.  Returns how many requests were queued.  This is what the
 * reference's scheduler does through extend_seq_list (vllm/core/scheduler.py:425-522 -> llama.py:328-337) for
 * callers that hold the segments but no scheduler: called every few steps with a distance of a few dozen rows,
 * no decode step maps a chunk in the calling thread. */
int vtkv_map_ahead_batch(vtkv_segment *const *segs, int n, int64_t ahead_bytes);
/* Map-ahead requests of the segment that are queued or running; 0 is the reference's "ready" flag
 * (query_shm, vmm_allocator.cpp:86-92). <0 on error. */
int vtkv_seg_pending(const vtkv_segment *s);
/* Wait until every map-ahead request has been carried out.  No counterpart in the reference. */
int vtkv_map_ahead_wait(void);

/* Batched bookkeeping of one model step; replaces extend_kv_cache_batch (vmm_allocator.h:138-168).
 * For i < n: if set_used_tokens[i] > 0, used = set_used_tokens[i]*kv_size; slot_m_out[i] = used;
 * then gen ? (ensure mapped, used += token_bytes[i]) : reserve(token_bytes[i], kv_size).
 * Unlike the reference the decode branch maps a chunk itself when the new token crosses the mapped
 * size (the reference leaves that to a racing background thread).  When the call fails (VTKV_ENOMEM: pool
 * exhausted) every segment's used size is what it was before the call, so the caller can preempt a
 * sequence and repeat the step; chunks mapped on the way stay mapped. */
int vtkv_extend_kv_cache_batch(vtkv_segment *const *segs, int n, const int64_t *token_bytes,
                               const int64_t *set_used_tokens, int64_t kv_size, int gen, int64_t *slot_m_out);

/* Device array of `num_seqs` base addresses; replaces KVCache(num_seqs) / getKVCachePtr
 * (vmm_allocator.cpp:458-470).  Returns a device address, 0 on error. */
uint64_t vtkv_ptr_table_create(int num_seqs);
int vtkv_ptr_table_destroy(uint64_t table);
/* table[slot] = ptr (synchronous); replaces KVCache::AddKVCache (vmm_allocator.cpp:463-466). */
int vtkv_ptr_table_set(uint64_t table, int slot, uint64_t ptr);
/* table[j] = K (which=0) or V (which=1) base of segs[j] for `layer`; replaces copy_kv_cache (vmm_allocator.h:170-182). */
int vtkv_ptr_table_fill(uint64_t table, vtkv_segment *const *segs, int n, int layer, int which);

/* Synchronous byte copies between host memory and any device address (mapped VMM ranges included).
 * For tests and debugging; replaces write_string / read_string (vmm_allocator.cpp:423-446). */
int vtkv_memcpy_h2d(uint64_t dst, const void *src, int64_t bytes);
int vtkv_memcpy_d2h(void *dst, uint64_t src, int64_t bytes);
/* Asynchronous upload on `stream` from pinned host memory (vtkv_host_alloc, or any hipHostMalloc'ed
 * buffer), which must stay untouched until the copy has run.  Carries a step's byte offsets and sequence
 * lengths to the device; replaces the torch.tensor(..., device="cuda") uploads of
 * vllm/model_executor/models/llama.py:340-341. */
int vtkv_memcpy_h2d_async(uint64_t dst, const void *src, int64_t bytes, void *stream);

/* ------------------------------------------------------------------------------------------
 * Cache ops.  Replace vllm._C.cache_ops (csrc/pybind.cpp:88-117, csrc/cache.h:8-44).
 * ---------------------------------------------------------------------------------------- */

/* vTensor scatter of new K/V rows; replaces reshape_and_cache (csrc/cache.h:18-29,
 * csrc/cache_kernels.cu:153-200,257-297).
 *   key,value      [num_tokens, num_heads, head_size] of src_dtype, row strides in elements
 *   k_ptrs,v_ptrs  device int64[max_seqs] base addresses (one per slot)
 *   slot_m         device int64[batch] byte offset of each sequence's next row (<0: skip)
 *   slot_ids       device int64[batch] slot of each sequence (python `slot_mapping`)
 *   seq_lens       device int32[batch] rows to write per sequence (ignored when max_seq_len == 1)
 *   cache_seq_lens device int32[batch] first source row of each sequence (ignored when max_seq_len == 1)
 * For sequence b, token t < max_seq_len: dst = ptrs[slot_ids[b]] + slot_m[b] + t*num_heads*head_size*e_kv,
 * src row = (max_seq_len == 1) ? b : cache_seq_lens[b] + t.
 * kv_dtype == src_dtype copies bits; kv_dtype == VTKV_FP8_E4M3 stores e4m3fn(x / scale) (round to
 * nearest even, saturating at +-448), slot_m is then in bytes of the fp8 range. */
int vtkv_reshape_and_cache(const void *key, const void *value, const int64_t *k_ptrs, const int64_t *v_ptrs,
                           const int64_t *slot_m, const int64_t *slot_ids, const int32_t *seq_lens,
                           const int32_t *cache_seq_lens, int batch, int max_seq_len, int num_heads, int head_size,
                           int64_t key_stride, int64_t value_stride, int src_dtype, int kv_dtype, float k_scale,
                           float v_scale, void *stream);

/* Upstream paged scatter, the layout the reference's kernel tests pin; replaces the 7-argument
 * reshape_and_cache (csrc/cpu/cache.cpp:103-128, tests/kernels/test_cache.py:115-193).
 * K cache [num_blocks, H, D/x, block_size, x], V cache [num_blocks, H, D, block_size], x = 16/elem_bytes;
 * slot_mapping device int64[num_tokens] (<0: skip). */
int vtkv_reshape_and_cache_paged(const void *key, const void *value, void *key_cache, void *value_cache,
                                 const int64_t *slot_mapping, int num_tokens, int num_heads, int head_size,
                                 int block_size, int64_t key_stride, int64_t value_stride, int elem_bytes,
                                 void *stream);

/* Copy whole blocks between two buffers; replaces swap_blocks (csrc/cache_kernels.cu:24-69).
 * `mapping` is a HOST int64[num_pairs,2] of (src_block, dst_block); one async copy of block_bytes per
 * maximal run of consecutive pairs, on `stream`.  Host buffers should be pinned. */
int vtkv_swap_blocks(const void *src, void *dst, int64_t block_bytes, const int64_t *mapping, int num_pairs,
                     int direction, void *stream);

/* Move `n` byte ranges (e.g. the mapped K and V ranges of swapped sequences) between device and pinned
 * host memory: every range is cut into pieces of at most piece_bytes (0 = default 16 MiB) that are dealt
 * round-robin to `num_streams` internal copy streams (<=8; 0 = default 2).  The copies start after the
 * work already queued on `stream` and `stream` waits for them to finish (event fork/join), so callers
 * keep ordinary stream semantics.  vTensor form of CacheEngine.swap_in/swap_out
 * (vllm/worker/cache_engine.py:131-139): the unit is a sequence's range, not a 16-token block. */
int vtkv_swap_ranges(const uint64_t *src, const uint64_t *dst, const int64_t *bytes, int n, int direction,
                     int64_t piece_bytes, int num_streams, void *stream);

/* Pinned host arena for swapped-out KV. */
void *vtkv_host_alloc(int64_t bytes);
int vtkv_host_free(void *p);

/* Scatter into the flash-attention cache layout; replaces reshape_and_cache_flash
 * (csrc/cache_kernels.cu:202-236,299-342; bound at csrc/pybind.cpp:100).  K and V caches are both
 * [num_blocks, block_size, H, D] with `block_stride` elements between blocks; slot_mapping device
 * int64[num_tokens] (<0: a padded token, skipped).  Unquantised caches only, as in the reference. */
int vtkv_reshape_and_cache_flash(const void *key, const void *value, void *k_cache, void *v_cache,
                                 const int64_t *slot_mapping, int num_tokens, int num_heads, int head_size,
                                 int block_size, int64_t block_stride, int64_t key_stride, int64_t value_stride,
                                 int elem_bytes, void *stream);

/* In-GPU block copies across layers; replaces copy_blocks (csrc/cache_kernels.cu:74-149).
 * key_caches/value_caches: HOST arrays of num_layers device base addresses (16-byte aligned; read before the
 * call returns, they travel as kernel arguments); `mapping`: DEVICE int64[num_pairs,2]; block_bytes must be a
 * multiple of 16.  Asynchronous on `stream`: no allocation, no upload, no wait. */
int vtkv_copy_blocks(const uint64_t *key_caches, const uint64_t *value_caches, int num_layers,
                     const int64_t *mapping, int num_pairs, int64_t block_bytes, void *stream);

/* Elementwise fp8 conversion; replaces convert_fp8 (csrc/cache_kernels.cu:346-422).
 * to_fp8 != 0: dst u8[n] = e4m3fn(src[n] / scale); else dst[n] = float(src u8[n]) * scale.
 * wide_dtype is the non-fp8 side (VTKV_F32, VTKV_BF16 or VTKV_F16). */
int vtkv_convert_fp8(void *dst, const void *src, int64_t n, float scale, int to_fp8, int wide_dtype, void *stream);

/* ------------------------------------------------------------------------------------------
 * Decode attention.  Replaces paged_attention_v1 / v2 (csrc/ops.h:6-19, csrc/attention/
 * attention_kernels.cu:85-448,608-737; split-K form :451-583) and the external fwd_kvcache
 * call (vllm/attention/backends/xformers.py:407-430).
 * ---------------------------------------------------------------------------------------- */

/* Bytes of scratch vtkv_decode_attention needs for these sizes (partition_tokens as below). */
int64_t vtkv_decode_attention_workspace_bytes(int num_seqs, int num_heads, int head_size, int max_seq_len,
                                              int partition_tokens);

/* out[b,h,:] = softmax(scale * q[b,h,:] . K_b^T [+ alibi]) V_b over the first seq_lens[b] rows of the
 * sequence's contiguous [T, num_kv_heads, head_size] K and V ranges, kv head = h / (num_heads/num_kv_heads).
 *   out        [num_seqs, num_heads, head_size] out_dtype, contiguous; out_dtype is q_dtype as in the
 *              reference, or VTKV_F32 to receive the result before its final rounding
 *   q          [num_seqs, num_heads, head_size] q_dtype, row stride q_stride elements
 *   k_ptrs,v_ptrs device int64[max_seqs]; slot_ids device int64[num_seqs]; seq_lens device int32[num_seqs]
 *   max_seq_len  host upper bound of seq_lens (sizes the grid, as in the reference launcher)
 *   alibi_slopes device float[num_heads] or NULL
 *   kv_dtype     q_dtype, or VTKV_FP8_E4M3 with k_scale / v_scale (x = code * scale)
 *   workspace    device scratch of at least vtkv_decode_attention_workspace_bytes(...) bytes, zero-filled by
 *                the caller before its first use and written by nobody else afterwards (the library keeps
 *                arrival counters in it and leaves them at zero after every call); calls that share a
 *                workspace must be ordered on one stream
 *   partition_tokens  0: the rows of the whole batch are cut into equal contiguous spans, one per
 *                workgroup of a grid that fills the device once, whatever the sequence lengths are;
 *                > 0 (a multiple of 16, at least 64): every workgroup takes that many rows, the
 *                reference's fixed partitions (512 in paged_attention_v2, csrc/attention/attention_kernels.cu:739-914).
 *                The result does not depend on the choice beyond fp32 summation order.
 * A launch takes up to 1024 sequences; a larger batch runs as consecutive launches of 1024 on `stream` within
 * the one call.
 * Supported: q_dtype VTKV_BF16 or VTKV_F16 with kv_dtype = q_dtype or VTKV_FP8_E4M3, head_size 64, 80, 96, 112, 128
 * or 256 (the reference's list, vllm/attention/ops/paged_attn.py:33-34), any whole num_heads/num_kv_heads.  The kernel
 * is tuned for bf16 and head size 128; the other shapes run the same code with their own tile constants.  A kv head
 * with more than 16 query heads (multi-query models) is served in ceil(n/16) parts of equal size (the last may be
 * smaller) that each read the kv head's rows: the parts count as kv heads towards the limit of 64 per call.
 * q_dtype VTKV_F32 (the reference's kernel tests also run float, tests/kernels/test_attention.py:23): float32 rows
 * and a float32 result (kv_dtype = out_dtype = VTKV_F32), every head size and head count, through a simpler kernel
 * of its own that computes in fp32 on the vector unit; partition_tokens is ignored (partitions of 512 rows, fewer
 * rows for small batches, more where the workspace does not hold the partial results); also through
 * vtkv_decode_attention_v2, vtkv_decode_attention_noalloc and vtkv_prefill_attention (where every prompt token
 * streams its own rows: right, and quadratic in HBM traffic), not through vtkv_decode_append_attention. */
int vtkv_decode_attention(void *out, const void *q, const int64_t *k_ptrs, const int64_t *v_ptrs,
                          const int64_t *slot_ids, const int32_t *seq_lens, int num_seqs, int num_heads,
                          int num_kv_heads, int head_size, int64_t q_stride, float scale, int max_seq_len,
                          const float *alibi_slopes, int q_dtype, int out_dtype, int kv_dtype, float k_scale,
                          float v_scale, void *workspace, int64_t workspace_bytes, int partition_tokens,
                          void *stream);

/* vtkv_decode_attention without a workspace argument and without any allocation.  No counterpart in the
 * reference: it is for callers that cannot allocate device memory around the call, i.e. code under HIP graph
 * capture, tight serving loops and harnesses that forbid hipMalloc.  The scratch (partial results, prefix sums,
 * arrival counters) is an array of vtkv_decode_attention_noalloc_max_bytes() = 32 MiB of device memory that is
 * part of the loaded library: every GPU the library runs on holds it until the process ends.  The call makes no
 * hipMalloc / hipFree and calls no allocating library routine; it launches the same kernels as
 * vtkv_decode_attention with partition_tokens = 0 and gives the same result bit for bit.  Sizes whose scratch
 * does not fit (roughly num_seqs * num_heads above 45 000) are refused with VTKV_EINVAL.  All calls on one GPU
 * share that GPU's array: calls that overlap in time on one GPU (two streams, two threads) race on it and must
 * be ordered by the caller; vtkv_set_kernel_timing does not apply to this entry point.
 * Under HIP graph capture: the first call on a device looks up the array's address and the kernels' occupancy
 * (hipGetSymbolAddress, an occupancy query), which are not stream work and must not happen while a stream is
 * capturing, so make one call on each device outside capture first; every later call only launches kernels (the
 * arrival counters are cleared by a kernel, not a memset) and can be recorded and replayed, with seq_lens read
 * from device memory at every replay. */
int64_t vtkv_decode_attention_noalloc_max_bytes(void);
int vtkv_decode_attention_noalloc(void *out, const void *q, const int64_t *k_ptrs, const int64_t *v_ptrs,
                                  const int64_t *slot_ids, const int32_t *seq_lens, int num_seqs, int num_heads,
                                  int num_kv_heads, int head_size, int64_t q_stride, float scale, int max_seq_len,
                                  const float *alibi_slopes, int q_dtype, int out_dtype, int kv_dtype, float k_scale,
                                  float v_scale, void *stream);

/* The reference's split-K interface: paged_attention_v2 (csrc/attention/attention_kernels.cu:451-583 kernel and
 * reduce, :739-914 launcher; CPU twin csrc/cpu/attention.cpp:434-646; Python vllm/attention/ops/paged_attn.py:
 * 139-166).  Same result as vtkv_decode_attention; the rows of every sequence are cut into partitions of 512,
 * one workgroup per (sequence, kv head, partition), and the caller's per-partition buffers are filled as the
 * reference fills them:
 *   exp_sums, max_logits  float [num_seqs, num_heads, max_num_partitions]: sum of exp(logit - max) over the
 *              partition's rows, and that max (scaled logits, natural units)
 *   tmp_out    [num_seqs, num_heads, max_num_partitions, head_size] of q_dtype: the partition's own normalised
 *              result
 *   max_num_partitions  >= ceil(max_seq_len / 512); entries of partitions past a sequence's end are not written
 * `out` is merged from the library's fp32 partials, not from the rounded tmp_out.
 * workspace: at least vtkv_decode_attention_v2_workspace_bytes(...) bytes, zero-filled before first use like
 * vtkv_decode_attention's (one buffer of the larger size can serve both). */
int64_t vtkv_decode_attention_v2_workspace_bytes(int num_seqs, int num_heads, int head_size, int max_num_partitions);
int vtkv_decode_attention_v2(void *out, float *exp_sums, float *max_logits, void *tmp_out, const void *q,
                             const int64_t *k_ptrs, const int64_t *v_ptrs, const int64_t *slot_ids,
                             const int32_t *seq_lens, int num_seqs, int num_heads, int num_kv_heads, int head_size,
                             int64_t q_stride, float scale, int max_seq_len, int max_num_partitions,
                             const float *alibi_slopes, int q_dtype, int out_dtype, int kv_dtype, float k_scale,
                             float v_scale, void *workspace, int64_t workspace_bytes, void *stream);

/* Query tokens one unit may hold (one workgroup per unit and kv head): 128 / g for head sizes up to 128, 64 / g for
 * 256, where g = num_heads/num_kv_heads, or, beyond 16, the heads of one of the ceil(g/16) parts a kv head is then
 * served in (71 heads: parts of 15).  0 for unsupported shapes.  vtkv_prefill_unit_tokens is the head size 128
 * form. */
int vtkv_prefill_unit_tokens_for(int num_heads, int num_kv_heads, int head_size, int kv_dtype);
int vtkv_prefill_unit_tokens(int num_heads, int num_kv_heads, int kv_dtype);

/* Causal attention of prompt (or chunked-prefill) tokens over the contiguous ranges, which already hold
 * the tokens' own rows (vtkv_reshape_and_cache runs first, as at vllm/attention/backends/xformers.py:
 * 301-312).  Replaces the prompt-run branch of the backend (xformers.py:331-386: the xformers call for a
 * plain prompt and the external fwd_kvcache call for a prompt with a cached prefix; both are the same
 * function of the cache contents).  The query token at position t of its sequence attends to rows 0..t.
 *   q, out   [num_query_tokens, num_heads, head_size]: the query tokens of all sequences, packed
 *   units    device int32[num_units][4] = {sequence index into slot_ids, first query row, number of query
 *            tokens (1 .. vtkv_prefill_unit_tokens_for(...)), position of the first of them in its sequence}:
 *            consecutive query tokens of one sequence that share one pass over its rows; every query
 *            token belongs to exactly one unit; longest units first balances the load best
 *   max_seq_len  host upper bound of position + 1 over all query tokens
 * No scratch is needed.  Other arguments as for vtkv_decode_attention.  Supported: head_size 64, 80, 96, 112, 128
 * or 256 (the kernel is tuned for 128; units hold vtkv_prefill_unit_tokens_for(...) tokens), q_dtype
 * VTKV_BF16 or VTKV_F16, kv_dtype = q_dtype or VTKV_FP8_E4M3 with k_scale / v_scale, out_dtype = q_dtype or
 * VTKV_F32; the longest-units-first order inside each sequence, sequence by sequence, lets every row be fetched
 * from HBM once.  q_dtype VTKV_F32 with kv_dtype = out_dtype = VTKV_F32 (float32 models): every token attends
 * through the float32 decode kernel by itself, without reuse of rows between tokens. */
int vtkv_prefill_attention(void *out, const void *q, const int64_t *k_ptrs, const int64_t *v_ptrs,
                           const int64_t *slot_ids, const int32_t *units, int num_units, int num_heads,
                           int num_kv_heads, int head_size, int64_t q_stride, float scale, int max_seq_len,
                           const float *alibi_slopes, int q_dtype, int out_dtype, int kv_dtype, float k_scale,
                           float v_scale, void *stream);

/* reshape_and_cache (decode form: one new row per sequence) fused into the attention launch; replaces
 * the pair of calls at vllm/attention/backends/xformers.py:310-312 and :357-371 for a decode step.
 * seq_lens[b] counts the new token: key[b] / value[b] ([num_seqs, num_kv_heads, head_size] of q_dtype, row strides
 * in elements) are appended at row seq_lens[b]-1 of sequence b's ranges, which must be mapped that far, and
 * attention runs over all seq_lens[b] rows.  The cache contents and the result are those of
 * vtkv_reshape_and_cache followed by vtkv_decode_attention (the result up to fp32 summation order).
 * Lengths come either from the device (seq_lens) or from the host (host_seq_lens: copied into the kernel
 * arguments during the call, 512 per launch, so no upload is needed and the array may be reused at once; a call
 * recorded into a HIP graph keeps the lengths it was recorded with, so a captured step passes device lengths);
 * pass NULL for the other.  q_dtype VTKV_BF16 or VTKV_F16 (the paired-head variants for very many short
 * sequences exist for bf16 at head size 128 only).  kv_dtype is q_dtype, or at head size 128 VTKV_FP8_E4M3 with
 * k_scale / v_scale: the new rows are then stored as e4m3fn(x / scale), bit for bit as vtkv_reshape_and_cache
 * stores them, and attended to in that form.  Head sizes 64, 80, 96, 112 and 256 take 16-bit caches
 * (VTKV_EINVAL for an fp8 cache: make the two calls).  Other arguments as for vtkv_decode_attention. */
int vtkv_decode_append_attention(void *out, const void *q, const void *key, const void *value, int64_t key_stride,
                                 int64_t value_stride, const int64_t *k_ptrs, const int64_t *v_ptrs,
                                 const int64_t *slot_ids, const int32_t *seq_lens, const int32_t *host_seq_lens,
                                 int num_seqs, int num_heads, int num_kv_heads, int head_size, int64_t q_stride,
                                 float scale, int max_seq_len, const float *alibi_slopes, int q_dtype, int out_dtype,
                                 int kv_dtype, float k_scale, float v_scale, void *workspace, int64_t workspace_bytes,
                                 int partition_tokens, void *stream);

/* Where the partial results of the workgroups that share a (sequence, kv head) are merged: 1 = inside the
 * attention kernel, by whichever of them finishes last; 0 = by a second kernel; -1 (the default) = inside
 * when the batch has at least two (sequence, kv head) pairs per workgroup (two and a half where the
 * head-major tile order does not apply), so that most need no merge.
 * For A/B measurements; results agree up to fp32 summation order.  No counterpart in the reference. */
int vtkv_set_fused_merge(int on);
/* Order in which the decode kernel's workgroups walk over the batch: 1 = (kv head, sequence, rows) wherever
 * the kernel supports it (no fixed partitions), 0 = (sequence, kv head, rows) always,
 * -1 (the default) = head-major where it lines the kv heads up with the eight XCDs (one contiguous eighth of
 * the order per XCD, and eight a multiple or a divisor of the kv heads, or pairs of fp8 kv heads, per sequence).
 * For A/B measurements; results agree up to fp32 summation order.  No counterpart in the reference. */
int vtkv_set_head_major(int on);

/* Benchmark aid without a counterpart in the reference (its kernel benchmark times from the host,
 * benchmarks/kernels/benchmark_paged_attention.py:147-157): while switched on, each vtkv_decode_attention
 * call (up to 1024 of them) launches its kernels with a start and a stop HIP event each on the caller's
 * stream (the begin and the end of that kernel's own dispatch, as a kernel trace reports them) without
 * waiting for them.  vtkv_attention_kernel_times waits for the recorded calls and writes, for the first
 * min(capacity, calls) of them in call order, the duration of the streaming kernel and of the merge
 * kernel in milliseconds (0 where the merge ran inside the streaming kernel); it returns that count.
 * Switching timing on again starts a new series. */
int vtkv_set_kernel_timing(int on);
int vtkv_attention_kernel_times(float *stream_ms, float *reduce_ms, int capacity);

#pragma GCC visibility pop
#ifdef __cplusplus
}
#endif
#endif /* VTKV_H */
