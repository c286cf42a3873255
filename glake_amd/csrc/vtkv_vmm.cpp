// Physical chunk pool and per-sequence virtual ranges on the HIP virtual-memory API.
//
// Each sequence slot owns, per layer, one K and one V address range reserved with
// hipMemAddressReserve; 2 MiB physical chunks created once with hipMemCreate are mapped at the
// end of the ranges as the sequence grows and go back to the pool when it is released, so KV of
// one sequence is always one contiguous [T, Hkv, D] array and kernels need no block table.
//
// Replaces the reference's vmm_allocator module (vmm_allocator/vmm_allocator.{h,cpp}).  What is
// deliberately different: one mutex guards the pool and every segment (the reference pops its
// request queue and touches the pool from two threads without a lock, vmm_allocator.cpp:43-48,
// 222-228); growth in the decode step is done in the calling thread instead of a detached busy-
// spinning thread signalling through POSIX shared memory (vmm_allocator.cpp:40-72,113-151);
// failed growth leaves the segment unchanged instead of half-mapped; the ranges of a destroyed segment
// are kept for the next segment of the same size and freed with the pool.
//
// Unmapping is lazy.  hipMemUnmap costs about 260 us per 2 MiB chunk on this hardware (mapping one
// costs about 55 us), so a segment that shrinks (preempt, release, swap-out) only gives its chunks
// up logically: they stay mapped at the top of its ranges as "retired" chunks, count as free, and
// are physically unmapped when another segment needs them (or when the caller asks with
// vtkv_pool_trim, e.g. while the GPU is busy).  If the same segment grows again first, as a sequence
// that is swapped back in or a slot that is reused does, its retired chunks are simply taken back
// without any call into the driver.
//
// Growth can also be requested ahead of need (vtkv_seg_eager_extend): a worker thread maps the chunks
// while the caller goes on, with the driver calls made outside the pool mutex, so the only thing that
// ever waits is an operation on the very segment that is being grown.  This is the reference's
// eagerExtend / eagerly_extend pair (vmm_allocator.cpp:40-72,307-320) with a condition variable in
// place of its busy-waiting thread and shared-memory flags, and with the request queue under the lock.
#include <algorithm>
#include <condition_variable>
#include <deque>
#include <mutex>
#include <thread>
#include <unordered_map>
#include <unordered_set>
#include <vector>

#include "vtkv_common.h"

namespace vtkv {

thread_local char g_err[512] = "";
char *error_buffer() { return g_err; }
int fail(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

namespace {

constexpr int64_t kMinChunk = 2ll << 20;  // vmm_allocator.h:45 granularitySize
// bytes of one physical chunk: the reference's 2 MiB unless vtkv_pool_set_chunk_bytes has asked for more
int64_t g_chunk = kMinChunk;

}  // namespace
}  // namespace vtkv
struct vtkv_segment;
namespace vtkv {
namespace {

struct Pool {
  std::mutex mu;
  int device = -1;
  std::vector<hipMemGenericAllocationHandle_t> free_chunks;
  int64_t total = 0;
  int64_t retired = 0;  // chunks still mapped at the top of shrunken segments; they count as free
  // chunks that are mapped into more than one segment (shared prefixes): handle -> number of mappings
  std::unordered_map<hipMemGenericAllocationHandle_t, int> shared;
  // mappings a chunk has been through since it was created, and their sum over all chunks of the pool
  // (see kRuntimeEntries)
  std::unordered_map<hipMemGenericAllocationHandle_t, int> cycles;
  int64_t pairs = 0;
  int64_t recreated = 0;
  // what the pool has asked of the runtime so far (reported when a mapping fails)
  int64_t maps = 0, ranges_reserved = 0, bytes_reserved = 0;
  // map-ahead worker (started on the first request, joined by vtkv_pool_destroy or at exit)
  struct Request { vtkv_segment *seg; int chunks; };
  std::deque<Request> requests;
  std::condition_variable work_cv, done_cv;
  std::thread worker;
  bool stop = false;
  ~Pool() {
    {
      std::unique_lock<std::mutex> lk(mu);
      stop = true;
    }
    work_cv.notify_all();
    if (worker.joinable()) worker.join();
  }
  std::unordered_set<vtkv_segment *> segments;
  // Address ranges of destroyed segments, by size, kept for the next segment of that size.  A range is
  // reserved once and freed when the pool is destroyed: with this runtime, freeing a range and reserving it
  // again leaves stale bookkeeping behind if the first incarnation had chunks mapped (seen as a crash
  // inside hipMemAddressFree of the second incarnation, and as hipMemMap failing with "invalid argument").
  // The reference never frees its ranges at all (vmm_allocator.cpp:177-212).
  std::unordered_map<int64_t, std::vector<char *>> spare_ranges;
};
Pool g_pool;

// An address range of `bytes` for a segment: a spare one of that size, else a new reservation.
hipError_t take_range_locked(int64_t bytes, char **out) {
  auto it = g_pool.spare_ranges.find(bytes);
  if (it != g_pool.spare_ranges.end() && !it->second.empty()) {
    *out = it->second.back();
    it->second.pop_back();
    return hipSuccess;
  }
  void *p = nullptr;
  const hipError_t e = hipMemAddressReserve(&p, bytes, g_chunk, nullptr, 0);
  *out = (char *)p;
  if (e == hipSuccess) {
    ++g_pool.ranges_reserved;
    g_pool.bytes_reserved += bytes;
  }
  return e;
}
void give_range_locked(char *p, int64_t bytes) { g_pool.spare_ranges[bytes].push_back(p); }

}  // namespace
}  // namespace vtkv

struct vtkv_segment {
  int layer_num = 0;
  int64_t context_max = 0;  // reserved bytes per range
  // The V rows start this many bytes into their range (the K rows at offset 0).  A wave reads the K and the V
  // row of the same token and kv head one after the other; with both ranges chunk-aligned the two requests
  // have the same address bits below 2 MiB and meet in the same memory channel, which costs 5 to 6 % of the
  // streaming rate (two arrays in lock step 6.6 to 6.7 TB/s, with 256 bytes between them 7.0 to 7.1, the
  // rate of one array).  Every mapping decision counts the offset: mapped >= used + v_skew.
  int64_t v_skew = 0;
  int64_t expand_bytes = 0; // what release keeps mapped
  int64_t mapped = 0;       // actual_size: bytes mapped per range that belong to the sequence
  int64_t held = 0;         // bytes physically mapped per range, >= mapped; [mapped, held) is retired
  int pending = 0;          // map-ahead requests queued or in progress; other changes of the segment wait
  int async_error = 0;      // a map-ahead request failed (reported by the next operation on the segment)
  int64_t used = 0;         // used_size: bytes written per range
  std::vector<char *> k_base, v_base;
  // chunks mapped into layer l's K (resp. V) range, in address order
  std::vector<std::vector<hipMemGenericAllocationHandle_t>> k_chunks, v_chunks;
};

using vtkv::g_pool;
using vtkv::g_chunk;

namespace {

void note_mapping_locked(hipMemGenericAllocationHandle_t h);  // below, with the rule it serves

// Map `n` chunks at offset `held` (== `mapped`: the caller has taken back all retired chunks) of
// every range.  Caller holds the pool mutex and has checked the free list holds 2*layers*n chunks.
// On a HIP failure everything mapped by this call is rolled back.
int map_chunks_locked(vtkv_segment *s, int n) {
  hipMemAccessDesc ad = {};
  ad.location.type = hipMemLocationTypeDevice;
  ad.location.id = g_pool.device;
  ad.flags = hipMemAccessFlagsProtReadWrite;
  struct Done { char *va; hipMemGenericAllocationHandle_t h; std::vector<hipMemGenericAllocationHandle_t> *list; };
  std::vector<Done> done;
  hipError_t err = hipSuccess;
  char where[128] = "";
  for (int l = 0; l < s->layer_num && err == hipSuccess; ++l) {
    for (int j = 0; j < n && err == hipSuccess; ++j) {
      for (int which = 0; which < 2 && err == hipSuccess; ++which) {
        char *va = (which ? s->v_base[l] : s->k_base[l]) + s->held + (int64_t)j * g_chunk;
        hipMemGenericAllocationHandle_t h = g_pool.free_chunks.back();
        err = hipMemMap(va, g_chunk, 0, h, 0);
        if (err != hipSuccess) {
          snprintf(where, sizeof(where), " (hipMemMap, %s range of layer %d, offset %lld of %lld)", which ? "V" : "K", l,
                   (long long)(s->held + (int64_t)j * g_chunk), (long long)s->context_max);
          break;
        }
        g_pool.free_chunks.pop_back();
        note_mapping_locked(h);
        auto *list = which ? &s->v_chunks[l] : &s->k_chunks[l];
        list->push_back(h);
        done.push_back({va, h, list});
        // (one call over several chunks costs the same per chunk: measured 28 us each either way)
        err = hipMemSetAccess(va, g_chunk, &ad, 1);
        if (err != hipSuccess)
          snprintf(where, sizeof(where), " (hipMemSetAccess, %s range of layer %d, offset %lld of %lld)", which ? "V" : "K",
                   l, (long long)(s->held + (int64_t)j * g_chunk), (long long)s->context_max);
      }
    }
  }
  if (err != hipSuccess) {
    for (auto it = done.rbegin(); it != done.rend(); ++it) {
      (void)hipMemUnmap(it->va, g_chunk);
      it->list->pop_back();
      g_pool.free_chunks.push_back(it->h);
    }
    return vtkv::fail(VTKV_EHIP, "mapping a chunk failed: %s%s; the pool has mapped %lld chunks (%lld mappings of its live chunks), "
                      "re-created %lld and reserved %lld ranges (%lld MiB) so far", hipGetErrorString(err), where,
                      (long long)g_pool.maps, (long long)g_pool.pairs, (long long)g_pool.recreated, (long long)g_pool.ranges_reserved,
                      (long long)(g_pool.bytes_reserved >> 20));
  }
  s->held += (int64_t)n * g_chunk;
  s->mapped = s->held;
  return VTKV_OK;
}

// This runtime keeps one entry per physical chunk and one per (chunk, virtual address) pair a chunk has
// ever been mapped at; it gives a pair's entry up only together with the chunk (hipMemRelease), and a
// process has 65 536 of them.  A pure HIP program with 700 chunks that maps one chunk at one of 1 200
// ranges per step, (chunk, range) pairs mostly new, gets "invalid argument" from hipMemSetAccess at step
// 64 810, and at step 63 510 with 2 000 chunks; with every chunk confined to two ranges it runs on without
// limit, and so it does when it re-creates a chunk every 16 or 64 mappings.  A server maps a chunk at a
// new address at every 2 MiB boundary a sequence crosses, so it would get there within hours.
//
// The pool therefore counts the mappings of every chunk since its creation (an upper bound of its pairs)
// and their sum, and re-creates a chunk when it comes back to the free list if the chunk has been through
// kCyclesPerChunk mappings or the sum is above the pool's share of the entries: above it every cycle of a
// chunk gives back at least the entry it took, so the sum stays below the share plus one entry per
// mapped chunk.  vtkv_pool_init keeps chunks + one pair per chunk below the limit.
constexpr int kCyclesPerChunk = 256;
constexpr int64_t kRuntimeEntries = 64000;   // of the 65 536: some are in use before the pool starts
constexpr int64_t kMaxPoolChunks = 30000;    // 2 entries per mapped chunk, and room to remap

int64_t pair_share_locked() { return std::max<int64_t>(kRuntimeEntries - 2 * g_pool.total - 1000, 2000); }

// `h` has just been mapped at an address.
void note_mapping_locked(hipMemGenericAllocationHandle_t h) {
  ++g_pool.cycles[h];
  ++g_pool.pairs;
  ++g_pool.maps;
}

// One mapping of `h` is gone: the chunk is free again unless another segment still maps it.
void release_handle_locked(hipMemGenericAllocationHandle_t h) {
  auto it = g_pool.shared.find(h);
  if (it != g_pool.shared.end()) {
    if (--it->second == 1) g_pool.shared.erase(it);
    return;
  }
  auto cyc = g_pool.cycles.find(h);
  const int n = cyc == g_pool.cycles.end() ? 0 : cyc->second;
  if (n > 0 && (n >= kCyclesPerChunk || g_pool.pairs > pair_share_locked())) {
    hipMemAllocationProp prop = {};
    prop.type = hipMemAllocationTypePinned;
    prop.location.type = hipMemLocationTypeDevice;
    prop.location.id = g_pool.device;
    hipMemGenericAllocationHandle_t fresh;
    // (if the new chunk cannot be had now, the old one serves on and is tried again after its next cycle)
    if (hipMemCreate(&fresh, g_chunk, &prop, 0) == hipSuccess) {
      g_pool.cycles.erase(cyc);
      g_pool.pairs -= n;
      (void)hipMemRelease(h);
      h = fresh;
      ++g_pool.recreated;
    }
  }
  g_pool.free_chunks.push_back(h);
}

// Physically unmap the retired chunks of `s` at offsets >= max(keep_held, mapped), top down, at most
// `max_rows` chunk rows (one row = one chunk of every range; < 0: all).  Returns rows unmapped or < 0.
int64_t trim_segment_locked(vtkv_segment *s, int64_t keep_held, int64_t max_rows) {
  const int64_t floor_n = std::max(keep_held, s->mapped) / g_chunk;
  int64_t rows = 0;
  while (s->held / g_chunk > floor_n && (max_rows < 0 || rows < max_rows)) {
    const int64_t top = s->held / g_chunk - 1;
    for (int l = 0; l < s->layer_num; ++l) {
      for (int which = 0; which < 2; ++which) {
        auto &list = which ? s->v_chunks[l] : s->k_chunks[l];
        char *base = which ? s->v_base[l] : s->k_base[l];
        // one call per mapping: each chunk was mapped on its own
        VTKV_HIP(hipMemUnmap(base + top * g_chunk, g_chunk));
        release_handle_locked(list.back());
        list.pop_back();
      }
    }
    s->held -= g_chunk;
    g_pool.retired -= 2ll * s->layer_num;
    ++rows;
  }
  return rows;
}

// Make the free list hold at least `need` chunks by unmapping retired chunks of other segments.
int reclaim_locked(int64_t need) {
  if ((int64_t)g_pool.free_chunks.size() >= need) return VTKV_OK;
  for (vtkv_segment *o : g_pool.segments) {
    while (o->held > o->mapped && (int64_t)g_pool.free_chunks.size() < need) {
      int64_t rc = trim_segment_locked(o, 0, 1);
      if (rc < 0) return (int)rc;
    }
    if ((int64_t)g_pool.free_chunks.size() >= need) return VTKV_OK;
  }
  return vtkv::fail(VTKV_ENOMEM, "chunk pool exhausted: need %lld, free %lld", (long long)need,
                    (long long)g_pool.free_chunks.size());
}

int expand_locked(vtkv_segment *s, int n) {
  if (n <= 0) return VTKV_OK;
  if (s->mapped + (int64_t)n * g_chunk > s->context_max)
    return vtkv::fail(VTKV_EINVAL, "segment would grow to %lld bytes, beyond its reserved %lld",
                      (long long)(s->mapped + (int64_t)n * g_chunk), (long long)s->context_max);
  // the segment's own retired chunks are still mapped right where it grows: take them back first
  const int revive = (int)std::min<int64_t>(n, (s->held - s->mapped) / g_chunk);
  const int fresh = n - revive;
  const int64_t need = 2ll * s->layer_num * fresh;
  // (its retired chunks beyond `revive` are none when fresh > 0, so reclaiming never touches `s`)
  if (fresh > 0 && (int64_t)g_pool.free_chunks.size() + g_pool.retired - 2ll * s->layer_num * revive < need)
    return vtkv::fail(VTKV_ENOMEM, "chunk pool exhausted: need %lld, free %lld", (long long)need,
                      (long long)((int64_t)g_pool.free_chunks.size() + g_pool.retired - 2ll * s->layer_num * revive));
  s->mapped += (int64_t)revive * g_chunk;
  g_pool.retired -= 2ll * s->layer_num * revive;
  if (fresh == 0) return VTKV_OK;
  int rc = reclaim_locked(need);
  if (rc >= 0) rc = map_chunks_locked(s, fresh);
  if (rc < 0) {  // leave the segment as it was
    s->mapped -= (int64_t)revive * g_chunk;
    g_pool.retired += 2ll * s->layer_num * revive;
  }
  return rc;
}

// Give up every chunk at offset >= keep_bytes of every range.  The chunks stay mapped (retired)
// until the pool needs them; see the note at the top of the file.
int shrink_locked(vtkv_segment *s, int64_t keep_bytes) {
  if (keep_bytes >= s->mapped) return VTKV_OK;
  const int64_t keep_n = keep_bytes / g_chunk;
  // Chunks that another segment maps as well cannot be counted as free while they sit here retired:
  // if any of the chunks given up is shared, everything above `keep` is unmapped right away.
  bool any_shared = false;
  if (!g_pool.shared.empty())
    for (int l = 0; l < s->layer_num && !any_shared; ++l)
      for (int which = 0; which < 2 && !any_shared; ++which) {
        const auto &list = which ? s->v_chunks[l] : s->k_chunks[l];
        for (int64_t j = keep_n; j < s->mapped / g_chunk && !any_shared; ++j) any_shared = g_pool.shared.count(list[j]) != 0;
      }
  g_pool.retired += 2ll * s->layer_num * (s->mapped / g_chunk - keep_n);
  s->mapped = keep_n * g_chunk;
  if (any_shared && trim_segment_locked(s, keep_bytes, -1) < 0) return VTKV_EHIP;
  return VTKV_OK;
}

// Wait until no map-ahead request of `s` is queued or running (the lock is released meanwhile).
void settle(std::unique_lock<std::mutex> &lk, vtkv_segment *s) {
  g_pool.done_cv.wait(lk, [&] { return s->pending == 0; });
}

// The map-ahead worker.  A request grows one segment by some chunks: retired chunks are taken back and
// handles for the rest are taken from the free list under the lock, the driver calls run without it,
// and the result is committed under the lock again.
void worker_main() {
  const bool device_ok = hipSetDevice(g_pool.device) == hipSuccess;
  std::unique_lock<std::mutex> lk(g_pool.mu);
  for (;;) {
    g_pool.work_cv.wait(lk, [] { return g_pool.stop || !g_pool.requests.empty(); });
    if (g_pool.stop) return;  // (vtkv_pool_destroy stops it with an empty queue; at exit requests are dropped)
    const auto rq = g_pool.requests.front();
    g_pool.requests.pop_front();
    vtkv_segment *s = rq.seg;
    if (!device_ok) {
      s->async_error = VTKV_EHIP;
      --s->pending;
      g_pool.done_cv.notify_all();
      continue;
    }
    int n = (int)std::min<int64_t>(rq.chunks, (s->context_max - s->mapped) / g_chunk);
    const int revive = (int)std::min<int64_t>(n, (s->held - s->mapped) / g_chunk);
    s->mapped += (int64_t)revive * g_chunk;
    g_pool.retired -= 2ll * s->layer_num * revive;
    n -= revive;
    const int64_t need = 2ll * s->layer_num * n;
    std::vector<hipMemGenericAllocationHandle_t> handles;
    if (n > 0 && reclaim_locked(need) >= 0) {
      handles.assign(g_pool.free_chunks.end() - need, g_pool.free_chunks.end());
      g_pool.free_chunks.resize(g_pool.free_chunks.size() - need);
    }
    if (n > 0 && handles.empty()) s->async_error = VTKV_ENOMEM;
    if (!handles.empty()) {
      const int64_t at = s->held;  // == mapped: nothing else changes the segment while it is pending
      const int layers = s->layer_num;
      lk.unlock();
      hipMemAccessDesc ad = {};
      ad.location.type = hipMemLocationTypeDevice;
      ad.location.id = g_pool.device;
      ad.flags = hipMemAccessFlagsProtReadWrite;
      hipError_t err = hipSuccess;
      size_t done = 0;  // handle index i maps range (layer, which) = (i / (2n), (i / n) % 2), chunk i % n
      auto va_of = [&](size_t i) {
        const int l = (int)(i / (2 * (size_t)n)), which = (int)((i / n) % 2), j = (int)(i % n);
        return (which ? s->v_base[l] : s->k_base[l]) + at + (int64_t)j * g_chunk;
      };
      for (; done < handles.size() && err == hipSuccess; ++done) {
        err = hipMemMap(va_of(done), g_chunk, 0, handles[done], 0);
        if (err != hipSuccess) break;
        err = hipMemSetAccess(va_of(done), g_chunk, &ad, 1);
        if (err != hipSuccess) {
          (void)hipMemUnmap(va_of(done), g_chunk);
          break;
        }
      }
      if (err != hipSuccess)
        for (size_t i = 0; i < done; ++i) (void)hipMemUnmap(va_of(i), g_chunk);
      lk.lock();
      for (size_t i = 0; i < std::min(done + 1, handles.size()); ++i) note_mapping_locked(handles[i]);
      if (err == hipSuccess) {
        for (int l = 0; l < layers; ++l)
          for (int which = 0; which < 2; ++which)
            for (int j = 0; j < n; ++j)
              (which ? s->v_chunks[l] : s->k_chunks[l]).push_back(handles[((size_t)l * 2 + which) * n + j]);
        s->held += (int64_t)n * g_chunk;
        s->mapped = s->held;
      } else {
        for (auto h : handles) g_pool.free_chunks.push_back(h);
        s->async_error = VTKV_EHIP;
      }
    }
    --s->pending;
    g_pool.done_cv.notify_all();
  }
}

int ensure_locked(vtkv_segment *s, int64_t token_bytes) {
  if (s->used + token_bytes + s->v_skew <= s->mapped) return 0;
  const int64_t gap = s->used + token_bytes + s->v_skew - s->mapped;
  const int n = (int)((gap + g_chunk - 1) / g_chunk);
  int rc = expand_locked(s, n);
  return rc < 0 ? rc : 1;
}

int reserve_locked(vtkv_segment *s, int64_t token_bytes, int64_t kv_size) {
  // vmm_allocator.cpp:322-337: room for the new rows plus a 100-row slack, rounded up to chunks
  const int64_t want = s->used + token_bytes + s->v_skew + 100 * kv_size;
  if (want > s->mapped) {
    int64_t n = (want - s->mapped + g_chunk - 1) / g_chunk;
    // the slack must not push a sequence past its reserved range
    const int64_t room = (s->context_max - s->mapped) / g_chunk;
    if (n > room) n = room;
    if (s->used + token_bytes + s->v_skew > s->mapped + n * g_chunk)
      return vtkv::fail(VTKV_EINVAL, "sequence of %lld bytes does not fit its reserved %lld",
                        (long long)(s->used + token_bytes), (long long)s->context_max);
    int rc = expand_locked(s, (int)n);
    if (rc < 0) return rc;
  }
  s->used += token_bytes;
  return VTKV_OK;
}

}  // namespace

extern "C" {

const char *vtkv_last_error(void) { return vtkv::error_buffer(); }
int vtkv_version(void) { return 100; }
int64_t vtkv_chunk_bytes(void) { return g_chunk; }

int vtkv_pool_set_chunk_bytes(int64_t bytes) {
  std::unique_lock<std::mutex> lk(g_pool.mu);
  VTKV_REQUIRE(bytes >= vtkv::kMinChunk && bytes <= (1ll << 30) && (bytes & (bytes - 1)) == 0,
               "chunk size %lld is not a power of two between 2 MiB and 1 GiB", (long long)bytes);
  if (bytes == g_chunk) return VTKV_OK;
  // chunks, segments and the kept address ranges are all laid out in units of the current size
  if (g_pool.total != 0 || !g_pool.segments.empty() || !g_pool.spare_ranges.empty())
    return vtkv::fail(VTKV_ESTATE, "the chunk size can only change while the pool is empty (before vtkv_pool_init "
                                   "or after vtkv_pool_destroy)");
  g_chunk = bytes;
  return VTKV_OK;
}

int vtkv_pool_init(int device, int64_t num_chunks) {
  std::unique_lock<std::mutex> lk(g_pool.mu);
  VTKV_REQUIRE(num_chunks >= 0, "num_chunks must be >= 0");
  if (g_pool.device >= 0 && g_pool.device != device)
    return vtkv::fail(VTKV_ESTATE, "pool already lives on device %d", g_pool.device);
  VTKV_HIP(hipSetDevice(device));
  int vmm = 0;
  VTKV_HIP(hipDeviceGetAttribute(&vmm, hipDeviceAttributeVirtualMemoryManagementSupported, device));
  if (!vmm) return vtkv::fail(VTKV_EHIP, "device %d has no virtual memory management support", device);
  hipMemAllocationProp prop = {};
  prop.type = hipMemAllocationTypePinned;
  prop.location.type = hipMemLocationTypeDevice;
  prop.location.id = device;
  size_t gran = 0;
  VTKV_HIP(hipMemGetAllocationGranularity(&gran, &prop, hipMemAllocationGranularityMinimum));
  if (gran == 0 || g_chunk % (int64_t)gran != 0)
    return vtkv::fail(VTKV_EHIP, "allocation granularity %zu does not divide the chunk size", gran);
  if (g_pool.total + num_chunks > kMaxPoolChunks)
    return vtkv::fail(VTKV_EINVAL,
                      "a pool of %lld chunks is more than this HIP runtime can serve: a process has 65536 entries for "
                      "chunks and (chunk, address) mappings together; at most %lld chunks (of %lld MiB; "
                      "vtkv_pool_set_chunk_bytes makes them larger)",
                      (long long)(g_pool.total + num_chunks), (long long)kMaxPoolChunks, (long long)(g_chunk >> 20));
  g_pool.device = device;
  g_pool.free_chunks.reserve(g_pool.free_chunks.size() + num_chunks);
  for (int64_t i = 0; i < num_chunks; ++i) {
    hipMemGenericAllocationHandle_t h;
    hipError_t e = hipMemCreate(&h, g_chunk, &prop, 0);
    if (e != hipSuccess)
      return vtkv::fail(VTKV_ENOMEM, "hipMemCreate failed after %lld of %lld chunks: %s", (long long)i,
                        (long long)num_chunks, hipGetErrorString(e));
    g_pool.free_chunks.push_back(h);
    ++g_pool.total;
  }
  return VTKV_OK;
}

int64_t vtkv_pool_free_chunks(void) {
  std::unique_lock<std::mutex> lk(g_pool.mu);
  return (int64_t)g_pool.free_chunks.size() + g_pool.retired;
}

int64_t vtkv_pool_recreated_chunks(void) {
  std::unique_lock<std::mutex> lk(g_pool.mu);
  return g_pool.recreated;
}

int64_t vtkv_pool_retired_chunks(void) {
  std::unique_lock<std::mutex> lk(g_pool.mu);
  return g_pool.retired;
}

int64_t vtkv_pool_trim(int64_t max_chunks) {
  std::unique_lock<std::mutex> lk(g_pool.mu);
  int64_t chunks = 0;
  for (vtkv_segment *s : g_pool.segments) {
    while (s->held > s->mapped && (max_chunks < 0 || chunks < max_chunks)) {
      int64_t rc = trim_segment_locked(s, 0, 1);
      if (rc < 0) return rc;
      chunks += 2ll * s->layer_num * rc;
    }
  }
  return chunks;
}

int64_t vtkv_pool_total_chunks(void) {
  std::unique_lock<std::mutex> lk(g_pool.mu);
  return g_pool.total;
}

int vtkv_pool_destroy(void) {
  std::unique_lock<std::mutex> lk(g_pool.mu);
  if (!g_pool.segments.empty())
    return vtkv::fail(VTKV_ESTATE, "%zu segments still alive", g_pool.segments.size());
  if (g_pool.worker.joinable()) {  // no segment is alive, so no request is queued
    g_pool.stop = true;
    g_pool.work_cv.notify_all();
    lk.unlock();
    g_pool.worker.join();
    lk.lock();
    g_pool.stop = false;
  }
  for (auto &kv : g_pool.spare_ranges)
    for (char *p : kv.second) VTKV_HIP(hipMemAddressFree(p, kv.first));
  g_pool.spare_ranges.clear();
  for (auto h : g_pool.free_chunks) VTKV_HIP(hipMemRelease(h));
  g_pool.free_chunks.clear();
  g_pool.cycles.clear();
  g_pool.pairs = 0;
  g_pool.total = 0;
  g_pool.device = -1;
  return VTKV_OK;
}

vtkv_segment *vtkv_seg_create(int layer_num, int64_t context_max_bytes, int64_t expand_bytes, int expand) {
  std::unique_lock<std::mutex> lk(g_pool.mu);
  if (g_pool.device < 0) {
    vtkv::fail(VTKV_ESTATE, "vtkv_pool_init has not been called");
    return nullptr;
  }
  if (layer_num <= 0 || context_max_bytes <= 0 || context_max_bytes % g_chunk != 0 || expand_bytes < 0 ||
      expand_bytes % g_chunk != 0 || expand_bytes > context_max_bytes) {
    vtkv::fail(VTKV_EINVAL, "layer_num must be > 0 and sizes multiples of the chunk size (max %lld, expand %lld)",
               (long long)context_max_bytes, (long long)expand_bytes);
    return nullptr;
  }
  auto *s = new vtkv_segment;
  s->layer_num = layer_num;
  s->context_max = context_max_bytes;
  s->expand_bytes = expand_bytes;
  s->k_chunks.resize(layer_num);
  s->v_chunks.resize(layer_num);
  auto unwind = [&](hipError_t e) {
    for (char *p : s->k_base) vtkv::give_range_locked(p, context_max_bytes);
    for (char *p : s->v_base) vtkv::give_range_locked(p, context_max_bytes);
    delete s;
    vtkv::fail(VTKV_EHIP, "hipMemAddressReserve failed: %s", hipGetErrorString(e));
    return (vtkv_segment *)nullptr;
  };
  for (int l = 0; l < layer_num; ++l) {
    char *k = nullptr, *v = nullptr;
    hipError_t e = vtkv::take_range_locked(context_max_bytes, &k);
    if (e != hipSuccess) return unwind(e);
    s->k_base.push_back(k);
    e = vtkv::take_range_locked(context_max_bytes, &v);
    if (e != hipSuccess) return unwind(e);
    s->v_base.push_back(v);
  }
  if (expand && expand_bytes > 0) {
    if (expand_locked(s, (int)(expand_bytes / g_chunk)) < 0) {
      for (char *p : s->k_base) vtkv::give_range_locked(p, context_max_bytes);
      for (char *p : s->v_base) vtkv::give_range_locked(p, context_max_bytes);
      delete s;
      return nullptr;
    }
  }
  g_pool.segments.insert(s);
  return s;
}

#define SEG_CHECK(s)                                                                                  \
  if (!(s) || !g_pool.segments.count(const_cast<vtkv_segment *>(s)))                                  \
  return vtkv::fail(VTKV_ESTATE, "not a live segment")

// Before a call that grows a segment: let its map-ahead requests finish, and report one that failed with a
// driver error (also when it failed a while ago and nothing is pending any more).  A request that found the
// pool empty is advisory only: it asked for a chunk ahead of need, the pool may have chunks again by now, and
// the call at hand maps what its own rows need and fails by itself if that cannot be had.
#define SEG_SETTLE(s)                                                                                 \
  do {                                                                                                \
    settle(lk, (s));                                                                                  \
    if ((s)->async_error) {                                                                           \
      const int e_ = (s)->async_error;                                                                \
      (s)->async_error = 0;                                                                           \
      if (e_ != VTKV_ENOMEM) return vtkv::fail(e_, "a map-ahead request of this segment failed (driver error)"); \
    }                                                                                                 \
  } while (0)
// Before a call that shrinks a segment (preempt, release, destroy): let its map-ahead requests finish and
// forget one that failed.  A full pool is exactly when the caller preempts to get chunks back, so these calls
// must do their work whatever became of a request to grow.
#define SEG_SETTLE_SHRINK(s)                                                                          \
  do {                                                                                                \
    settle(lk, (s));                                                                                  \
    (s)->async_error = 0;                                                                             \
  } while (0)

int vtkv_seg_destroy(vtkv_segment *s) {
  std::unique_lock<std::mutex> lk(g_pool.mu);
  SEG_CHECK(s);
  SEG_SETTLE_SHRINK(s);
  int rc = shrink_locked(s, 0);
  if (rc < 0) return rc;
  if (trim_segment_locked(s, 0, -1) < 0) return VTKV_EHIP;
  // every chunk is unmapped; the ranges wait for the next segment of this size
  for (char *p : s->k_base) vtkv::give_range_locked(p, s->context_max);
  for (char *p : s->v_base) vtkv::give_range_locked(p, s->context_max);
  g_pool.segments.erase(s);
  delete s;
  return VTKV_OK;
}

uint64_t vtkv_seg_key_ptr(const vtkv_segment *s, int layer) {
  std::unique_lock<std::mutex> lk(g_pool.mu);
  if (!s || !g_pool.segments.count(const_cast<vtkv_segment *>(s)) || layer < 0 || layer >= s->layer_num) {
    vtkv::fail(VTKV_EINVAL, "bad segment or layer %d", layer);
    return 0;
  }
  return (uint64_t)(uintptr_t)s->k_base[layer];
}

uint64_t vtkv_seg_value_ptr(const vtkv_segment *s, int layer) {
  std::unique_lock<std::mutex> lk(g_pool.mu);
  if (!s || !g_pool.segments.count(const_cast<vtkv_segment *>(s)) || layer < 0 || layer >= s->layer_num) {
    vtkv::fail(VTKV_EINVAL, "bad segment or layer %d", layer);
    return 0;
  }
  return (uint64_t)(uintptr_t)(s->v_base[layer] + s->v_skew);
}

int64_t vtkv_seg_value_skew(const vtkv_segment *s) {
  std::unique_lock<std::mutex> lk(g_pool.mu);
  SEG_CHECK(s);
  return s->v_skew;
}

int vtkv_seg_set_value_skew(vtkv_segment *s, int64_t bytes) {
  std::unique_lock<std::mutex> lk(g_pool.mu);
  SEG_CHECK(s);
  VTKV_REQUIRE(bytes >= 0 && bytes <= 4096 && bytes % 256 == 0, "value skew %lld is not a multiple of 256 in [0, 4096]",
               (long long)bytes);
  if (s->used != 0) return vtkv::fail(VTKV_ESTATE, "the value skew can only change while the segment holds no rows");
  s->v_skew = bytes;
  return VTKV_OK;
}

int64_t vtkv_seg_get_used(const vtkv_segment *s) {
  std::unique_lock<std::mutex> lk(g_pool.mu);
  SEG_CHECK(s);
  return s->used;
}

int vtkv_seg_set_used(vtkv_segment *s, int64_t used) {
  std::unique_lock<std::mutex> lk(g_pool.mu);
  SEG_CHECK(s);
  VTKV_REQUIRE(used >= 0 && used <= s->context_max - s->v_skew, "used_bytes %lld outside [0, %lld]", (long long)used,
               (long long)(s->context_max - s->v_skew));
  s->used = used;
  return VTKV_OK;
}

int64_t vtkv_seg_mapped_bytes(const vtkv_segment *s) {
  std::unique_lock<std::mutex> lk(g_pool.mu);
  SEG_CHECK(s);
  return s->mapped;
}

int vtkv_seg_expand(vtkv_segment *s, int n) {
  std::unique_lock<std::mutex> lk(g_pool.mu);
  SEG_CHECK(s);
  SEG_SETTLE(s);
  VTKV_REQUIRE(n >= 0, "num_chunks must be >= 0");
  return expand_locked(s, n);
}

int vtkv_seg_reserve(vtkv_segment *s, int64_t token_bytes, int64_t kv_size) {
  std::unique_lock<std::mutex> lk(g_pool.mu);
  SEG_CHECK(s);
  SEG_SETTLE(s);
  VTKV_REQUIRE(token_bytes >= 0 && kv_size >= 0, "sizes must be >= 0");
  return reserve_locked(s, token_bytes, kv_size);
}

int vtkv_seg_ensure(vtkv_segment *s, int64_t token_bytes) {
  std::unique_lock<std::mutex> lk(g_pool.mu);
  SEG_CHECK(s);
  SEG_SETTLE(s);
  VTKV_REQUIRE(token_bytes >= 0, "token_bytes must be >= 0");
  return ensure_locked(s, token_bytes);
}

int vtkv_seg_preempt(vtkv_segment *s) {
  std::unique_lock<std::mutex> lk(g_pool.mu);
  SEG_CHECK(s);
  SEG_SETTLE_SHRINK(s);
  int rc = shrink_locked(s, 0);
  if (rc < 0) return rc;
  s->used = 0;
  return VTKV_OK;
}

int vtkv_seg_release(vtkv_segment *s) {
  std::unique_lock<std::mutex> lk(g_pool.mu);
  SEG_CHECK(s);
  SEG_SETTLE_SHRINK(s);
  // vmm_allocator.cpp:393-420: keep the first expand_size bytes mapped when at least that much is
  // mapped, otherwise (fewer bytes mapped than expand_size) unmap everything.
  const int64_t keep = s->mapped >= s->expand_bytes ? s->expand_bytes : 0;
  int rc = shrink_locked(s, keep);
  if (rc < 0) return rc;
  s->used = 0;
  return VTKV_OK;
}

int vtkv_seg_share_prefix(vtkv_segment *dst, vtkv_segment *src, int64_t bytes, void *stream) {
  std::unique_lock<std::mutex> lk(g_pool.mu);
  SEG_CHECK(dst);
  SEG_CHECK(src);
  SEG_SETTLE(dst);
  settle(lk, src);  // the source is not changed: a failed request of its own is its next growth call's to report
  VTKV_REQUIRE(dst != src && dst->layer_num == src->layer_num, "segments must differ and have the same layer count");
  VTKV_REQUIRE(bytes >= 0 && bytes <= src->used && src->used <= src->mapped, "prefix of %lld bytes exceeds the source's %lld",
               (long long)bytes, (long long)src->used);
  VTKV_REQUIRE(dst->mapped == 0 && dst->used == 0, "the destination segment must be empty");
  // A chunk is shared only if the prefix fills it in the K range (there the V range, whose rows lie v_skew
  // bytes further on, is filled by the prefix as well); what lies behind the whole chunks, up to the end of
  // the prefix's V rows, is the tail, copied into one or two chunks of the destination's own.
  VTKV_REQUIRE(dst->v_skew == src->v_skew, "the segments place their V rows differently");
  const int64_t skew = src->v_skew;
  const int64_t whole = bytes / g_chunk, tail = bytes ? bytes + skew - whole * g_chunk : 0;
  const int64_t own = (tail + g_chunk - 1) / g_chunk;
  VTKV_REQUIRE((whole + own) * g_chunk <= dst->context_max, "prefix does not fit the destination's range");
  VTKV_REQUIRE(bytes == 0 || bytes + skew <= src->mapped, "the source's mapping ends inside the prefix");
  if (trim_segment_locked(dst, 0, -1) < 0) return VTKV_EHIP;  // its retired chunks would be in the way
  if ((int64_t)g_pool.free_chunks.size() + g_pool.retired < own * 2ll * dst->layer_num)
    return vtkv::fail(VTKV_ENOMEM, "chunk pool exhausted: need %lld, free %lld", own * 2ll * dst->layer_num,
                      (long long)((int64_t)g_pool.free_chunks.size() + g_pool.retired));
  // whole chunks: the same physical chunk at the same offset of the destination's range
  hipMemAccessDesc ad = {};
  ad.location.type = hipMemLocationTypeDevice;
  ad.location.id = g_pool.device;
  ad.flags = hipMemAccessFlagsProtReadWrite;
  struct Done { char *va; std::vector<hipMemGenericAllocationHandle_t> *list; hipMemGenericAllocationHandle_t h; };
  std::vector<Done> done;
  hipError_t err = hipSuccess;
  for (int l = 0; l < dst->layer_num && err == hipSuccess; ++l)
    for (int which = 0; which < 2 && err == hipSuccess; ++which) {
      auto &from = which ? src->v_chunks[l] : src->k_chunks[l];
      auto &to = which ? dst->v_chunks[l] : dst->k_chunks[l];
      char *base = which ? dst->v_base[l] : dst->k_base[l];
      for (int64_t j = 0; j < whole && err == hipSuccess; ++j) {
        char *va = base + j * g_chunk;
        err = hipMemMap(va, g_chunk, 0, from[j], 0);
        if (err != hipSuccess) break;
        note_mapping_locked(from[j]);
        to.push_back(from[j]);
        done.push_back({va, &to, from[j]});
        err = hipMemSetAccess(va, g_chunk, &ad, 1);
      }
    }
  if (err != hipSuccess) {
    for (auto it = done.rbegin(); it != done.rend(); ++it) {
      (void)hipMemUnmap(it->va, g_chunk);
      it->list->pop_back();
    }
    return vtkv::fail(VTKV_EHIP, "mapping a shared chunk failed: %s", hipGetErrorString(err));
  }
  for (const Done &d : done) {
    auto it = g_pool.shared.find(d.h);
    if (it == g_pool.shared.end()) g_pool.shared[d.h] = 2; else ++it->second;
  }
  dst->held = dst->mapped = whole * g_chunk;
  if (tail) {
    // the partly filled chunk is the destination's own: both sequences go on writing behind the prefix
    int rc = expand_locked(dst, (int)own);
    if (rc < 0) {
      (void)shrink_locked(dst, 0);
      return rc;
    }
    for (int l = 0; l < dst->layer_num; ++l)
      for (int which = 0; which < 2; ++which) {
        char *to = (which ? dst->v_base[l] : dst->k_base[l]) + whole * g_chunk;
        const char *from = (which ? src->v_base[l] : src->k_base[l]) + whole * g_chunk;
        const int64_t n = which ? tail : tail - skew;  // the K rows end that much before the V rows
        if (n > 0) VTKV_HIP(hipMemcpyAsync(to, from, (size_t)n, hipMemcpyDeviceToDevice, (hipStream_t)stream));
      }
  }
  dst->used = bytes;
  return VTKV_OK;
}

int64_t vtkv_pool_shared_chunks(void) {
  std::unique_lock<std::mutex> lk(g_pool.mu);
  return (int64_t)g_pool.shared.size();
}

int vtkv_seg_eager_extend(vtkv_segment *s, int num_chunks) {
  std::unique_lock<std::mutex> lk(g_pool.mu);
  SEG_CHECK(s);
  VTKV_REQUIRE(num_chunks >= 0, "num_chunks must be >= 0");
  if (num_chunks == 0 || s->mapped >= s->context_max) return VTKV_OK;  // vmm_allocator.cpp:310: nothing left to map
  if (!g_pool.worker.joinable()) g_pool.worker = std::thread(worker_main);
  ++s->pending;
  g_pool.requests.push_back({s, num_chunks});
  g_pool.work_cv.notify_one();
  return VTKV_OK;
}

int vtkv_map_ahead_batch(vtkv_segment *const *segs, int n, int64_t ahead_bytes) {
  std::unique_lock<std::mutex> lk(g_pool.mu);
  VTKV_REQUIRE(n >= 0 && (n == 0 || segs) && ahead_bytes >= 0, "bad segment list or distance");
  for (int i = 0; i < n; ++i) SEG_CHECK(segs[i]);
  // only what the pool can serve now is asked for: a request that fails is reported by the segment's next
  // growth, and a sequence may finish before it needs the chunk
  int64_t spare = (int64_t)g_pool.free_chunks.size() + g_pool.retired;
  // chunks that requests still in the queue will take (earlier calls, vtkv_seg_eager_extend) are spoken for;
  // counted in full, a retired chunk a request may revive instead only makes the estimate more careful
  for (const auto &rq : g_pool.requests) spare -= 2ll * rq.seg->layer_num * rq.chunks;
  int queued = 0;
  for (int i = 0; i < n; ++i) {
    vtkv_segment *s = segs[i];
    if (s->async_error == VTKV_ENOMEM) s->async_error = 0;  // an earlier request found the pool empty: ask again
    if (s->pending || s->async_error || s->mapped >= s->context_max) continue;
    if (s->used + s->v_skew + ahead_bytes <= s->mapped) continue;
    const int64_t revive = s->held > s->mapped ? 1 : 0;  // a retired chunk of its own comes back without a driver call
    const int64_t need = revive ? 0 : 2ll * s->layer_num;
    if (spare < need) continue;
    spare -= need;
    if (!g_pool.worker.joinable()) g_pool.worker = std::thread(worker_main);
    ++s->pending;
    g_pool.requests.push_back({s, 1});
    ++queued;
  }
  if (queued) g_pool.work_cv.notify_one();
  return queued;
}

int vtkv_seg_pending(const vtkv_segment *s) {
  std::unique_lock<std::mutex> lk(g_pool.mu);
  SEG_CHECK(s);
  return s->pending;
}

int vtkv_map_ahead_wait(void) {
  std::unique_lock<std::mutex> lk(g_pool.mu);
  g_pool.done_cv.wait(lk, [] {
    if (!g_pool.requests.empty()) return false;
    for (vtkv_segment *s : g_pool.segments)
      if (s->pending) return false;
    return true;
  });
  return VTKV_OK;
}

int vtkv_extend_kv_cache_batch(vtkv_segment *const *segs, int n, const int64_t *token_bytes,
                               const int64_t *set_used_tokens, int64_t kv_size, int gen, int64_t *slot_m_out) {
  std::unique_lock<std::mutex> lk(g_pool.mu);
  VTKV_REQUIRE(n >= 0 && (n == 0 || (segs && token_bytes && slot_m_out)), "null argument");
  for (int i = 0; i < n; ++i) SEG_CHECK(segs[i]);
  // A failure part of the way through (pool exhausted, a failed map-ahead request) leaves every sequence's used
  // size as it was before the call, so that the caller can preempt a sequence and run the step again; chunks
  // mapped on the way stay mapped.
  std::vector<int64_t> before((size_t)n);
  for (int i = 0; i < n; ++i) before[(size_t)i] = segs[i]->used;
  auto body = [&]() -> int {
    for (int i = 0; i < n; ++i) {
      vtkv_segment *s = segs[i];
      if (set_used_tokens && set_used_tokens[i] > 0) s->used = set_used_tokens[i] * kv_size;
      // rows that need a chunk which is being mapped ahead wait for it here (a prompt always does: its
      // reservation looks 100 rows ahead); a request that failed earlier is reported by this call too
      if ((s->pending && (!gen || s->used + token_bytes[i] + s->v_skew > s->mapped)) || (!s->pending && s->async_error))
        SEG_SETTLE(s);
      slot_m_out[i] = s->used;
      if (gen) {
        int rc = ensure_locked(s, token_bytes[i]);
        if (rc < 0) return rc;
        s->used += token_bytes[i];
      } else {
        int rc = reserve_locked(s, token_bytes[i], kv_size);
        if (rc < 0) return rc;
      }
    }
    return VTKV_OK;
  };
  const int rc = body();
  if (rc < 0)
    for (int i = 0; i < n; ++i) segs[i]->used = before[(size_t)i];
  return rc;
}

uint64_t vtkv_ptr_table_create(int num_seqs) {
  if (num_seqs <= 0) {
    vtkv::fail(VTKV_EINVAL, "num_seqs must be > 0");
    return 0;
  }
  void *p = nullptr;
  hipError_t e = hipMalloc(&p, (size_t)num_seqs * sizeof(uint64_t));
  if (e != hipSuccess) {
    vtkv::fail(VTKV_EHIP, "hipMalloc failed: %s", hipGetErrorString(e));
    return 0;
  }
  (void)hipMemset(p, 0, (size_t)num_seqs * sizeof(uint64_t));
  return (uint64_t)(uintptr_t)p;
}

int vtkv_ptr_table_destroy(uint64_t table) {
  VTKV_HIP(hipFree((void *)(uintptr_t)table));
  return VTKV_OK;
}

int vtkv_ptr_table_set(uint64_t table, int slot, uint64_t ptr) {
  VTKV_REQUIRE(table != 0 && slot >= 0, "bad table or slot");
  VTKV_HIP(hipMemcpy((char *)(uintptr_t)table + (size_t)slot * 8, &ptr, 8, hipMemcpyHostToDevice));
  return VTKV_OK;
}

int vtkv_ptr_table_fill(uint64_t table, vtkv_segment *const *segs, int n, int layer, int which) {
  std::vector<uint64_t> host(n > 0 ? n : 0);
  {
    std::unique_lock<std::mutex> lk(g_pool.mu);
    VTKV_REQUIRE(table != 0 && n >= 0 && (n == 0 || segs), "bad table or segment list");
    for (int i = 0; i < n; ++i) {
      SEG_CHECK(segs[i]);
      VTKV_REQUIRE(layer >= 0 && layer < segs[i]->layer_num, "layer %d out of range", layer);
      host[i] = (uint64_t)(uintptr_t)(which ? segs[i]->v_base[layer] + segs[i]->v_skew : segs[i]->k_base[layer]);
    }
  }
  if (n > 0) VTKV_HIP(hipMemcpy((void *)(uintptr_t)table, host.data(), (size_t)n * 8, hipMemcpyHostToDevice));
  return VTKV_OK;
}

int vtkv_memcpy_h2d(uint64_t dst, const void *src, int64_t bytes) {
  VTKV_REQUIRE(bytes >= 0 && (bytes == 0 || (dst && src)), "null argument");
  if (bytes) VTKV_HIP(hipMemcpy((void *)(uintptr_t)dst, src, (size_t)bytes, hipMemcpyHostToDevice));
  return VTKV_OK;
}

int vtkv_memcpy_h2d_async(uint64_t dst, const void *src, int64_t bytes, void *stream) {
  VTKV_REQUIRE(bytes >= 0 && (bytes == 0 || (dst && src)), "null argument");
  if (bytes)
    VTKV_HIP(hipMemcpyAsync((void *)(uintptr_t)dst, src, (size_t)bytes, hipMemcpyHostToDevice, (hipStream_t)stream));
  return VTKV_OK;
}

int vtkv_memcpy_d2h(void *dst, uint64_t src, int64_t bytes) {
  VTKV_REQUIRE(bytes >= 0 && (bytes == 0 || (dst && src)), "null argument");
  if (bytes) VTKV_HIP(hipMemcpy(dst, (const void *)(uintptr_t)src, (size_t)bytes, hipMemcpyDeviceToHost));
  return VTKV_OK;
}

void *vtkv_host_alloc(int64_t bytes) {
  void *p = nullptr;
  if (bytes <= 0) {
    vtkv::fail(VTKV_EINVAL, "bytes must be > 0");
    return nullptr;
  }
  hipError_t e = hipHostMalloc(&p, (size_t)bytes, hipHostMallocDefault);
  if (e != hipSuccess) {
    vtkv::fail(VTKV_EHIP, "hipHostMalloc(%lld) failed: %s", (long long)bytes, hipGetErrorString(e));
    return nullptr;
  }
  return p;
}

int vtkv_host_free(void *p) {
  if (p) VTKV_HIP(hipHostFree(p));
  return VTKV_OK;
}

}  // extern "C"
