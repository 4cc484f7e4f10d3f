// Thin HIP device API behind DLArrayAlloc / DLArrayFree / DLArrayCopyFromTo and
// the stream / handle factories.
//
// Replaces the reference's DeviceAPIManager + CUDADeviceAPI + CPUDeviceAPI
// (src/c_runtime_api.cc:21-164, src/cuda_device_api.cc:22-81,
// src/cpu_device_api.cc:12-36).  Differences that are deliberate:
//   * device and pinned-host storage come from a caching allocator, so the
//     executor's allocate-per-node-per-step pattern (pycode/tinyflow/autodiff.py:2778)
//     costs a map lookup instead of a hipMalloc/hipFree pair;
//   * ops do not block the host; copies order themselves after enqueued work.
#include "internal.h"

#include <atomic>
#include <cstring>
#include <map>
#include <mutex>
#include <unordered_map>
#include <vector>

namespace tf {
namespace {

struct StreamRec {
  hipStream_t stream;
  hipEvent_t event;   // reusable marker for cross-stream ordering
  bool runs_kernels;  // an op entry point has launched on it (copy-only streams stay false)
  unsigned *fold_tickets = nullptr;  // counters of the contraction kernels' in-kernel fold (see fold_tickets)
};

__global__ void zero_words_kernel(unsigned *p, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0u;
}

struct Runtime {
  std::mutex mu;
  // caching allocator state (one per memory kind)
  struct Pool {
    std::multimap<size_t, void *> free_blocks;      // size -> block
    std::unordered_map<void *, size_t> block_size;  // every block obtained from HIP
    size_t reserved = 0;                            // bytes held from HIP (in use + cached)
    size_t in_use = 0;                              // bytes handed out and not yet returned
    size_t peak_in_use = 0;
  };
  Pool dev, host;
  size_t dev_limit = 0;  // 0 = unlimited; TINYFLOW_GPU_MEM_LIMIT_MB

  // Under a budget, device memory comes from one arena obtained with a single
  // hipMalloc and sub-allocated best-fit with coalescing: a step that runs at the
  // budget then never calls hipMalloc / hipFree (hipFree waits for the whole
  // device, which would stall the copy streams of the swap path on every
  // allocation).  Blocks handed out before the budget was set stay with `dev`.
  struct Arena {
    char *base = nullptr;
    size_t size = 0, used_bytes = 0;
    bool retired = false;                        // budget changed: serve no new requests
    std::map<size_t, size_t> free_by_off;        // offset -> length
    std::multimap<size_t, size_t> free_by_len;   // length -> offset
    // release fences by address: non-overlapping segments covering the arena, each with the
    // fence of the last release that touched it (free ranges coalesce, their histories must not:
    // a merged range would inherit its youngest neighbour's fence)
    struct Seg { size_t len; uint64_t fence; };
    std::map<size_t, Seg> fence_seg;             // offset -> segment
    std::unordered_map<void *, size_t> used;     // pointer -> length
  } arena;
  // Release fences.  Every device block remembers the number of the first fence
  // recorded, on the kernel-running stream, after its storage was last given back:
  // all kernels that could still touch the storage were enqueued before that
  // fence.  A release only notes the number of the next fence (fence_count + 1);
  // the event itself is recorded when somebody asks for it (DLArrayPrepareFresh), so
  // releases cost nothing and a step records one event per prefetch.  Fences live in
  // a ring of events; a slot that has been reused holds a later fence of the same
  // stream, which is just as safe to wait for.
  static constexpr int kFenceRing = 1024;
  static constexpr uint64_t kNoFence = 0;                  // storage never handed back since it came from HIP
  static constexpr uint64_t kConservative = ~(uint64_t)0;  // no single stream to fence on: wait for all
  hipEvent_t fence_ring[kFenceRing] = {};
  uint64_t fence_count = 0;
  std::unordered_map<void *, uint64_t> pool_fence;   // cached / handed-out pool block -> fence of its last release
  std::unordered_map<void *, uint64_t> block_fence;  // handed-out device block -> fence to honour before reuse
  std::vector<StreamRec> streams;
  bool sync_ops = false;
  int cus = 0;
  bool inited = false;

  void init() {
    if (inited) return;
    inited = true;
    if (const char *e = getenv("TINYFLOW_GPU_MEM_LIMIT_MB")) dev_limit = (size_t)atoll(e) << 20;
    if (const char *e = getenv("TINYFLOW_SYNC_EVERY_OP")) sync_ops = atoi(e) != 0;
  }
};

Runtime &rt() {
  static Runtime *r = new Runtime();  // leaked on purpose: arrays may be freed during interpreter exit
  return *r;
}

size_t round_size(size_t bytes) {
  if (bytes == 0) bytes = 1;
  const size_t q = bytes < (1u << 20) ? 512 : (size_t)1 << 16;  // 512 B below 1 MiB, 64 KiB above
  return (bytes + q - 1) / q * q;
}

// Give cached blocks of `p` back to HIP, largest first, until `need` more bytes fit
// under `limit` (everything when limit == 0).  hipFree waits for the device, so
// blocks still referenced by enqueued kernels are safe to release.
void release_cached(Runtime::Pool &p, bool device, size_t need, size_t limit) {
  while (!p.free_blocks.empty()) {
    if (limit != 0 && p.reserved + need <= limit) break;
    auto it = std::prev(p.free_blocks.end());
    if (device) {
      (void)hipFree(it->second);
      rt().pool_fence.erase(it->second);
    } else {
      (void)hipHostFree(it->second);
    }
    p.reserved -= it->first;
    p.block_size.erase(it->second);
    p.free_blocks.erase(it);
  }
}

void arena_erase_free(Runtime::Arena &a, size_t off, size_t len) {
  a.free_by_off.erase(off);
  auto range = a.free_by_len.equal_range(len);
  for (auto it = range.first; it != range.second; ++it)
    if (it->second == off) {
      a.free_by_len.erase(it);
      break;
    }
}

void arena_insert_free(Runtime::Arena &a, size_t off, size_t len) {
  a.free_by_off[off] = len;
  a.free_by_len.emplace(len, off);
}

// Fence numbers grow along the one stream they are recorded on, so the later of two is the larger.
uint64_t later_fence(uint64_t x, uint64_t y) { return x > y ? x : y; }

// Stamps [off, off + len) with `fence`, splitting the segments it overlaps.
void arena_set_fence(Runtime::Arena &a, size_t off, size_t len, uint64_t fence) {
  const size_t end = off + len;
  auto it = a.fence_seg.upper_bound(off);
  if (it != a.fence_seg.begin()) --it;
  while (it != a.fence_seg.end() && it->first < end) {
    const size_t s_off = it->first, s_end = it->first + it->second.len;
    const uint64_t s_fence = it->second.fence;
    if (s_end <= off) {
      ++it;
      continue;
    }
    it = a.fence_seg.erase(it);
    if (s_off < off) a.fence_seg[s_off] = {off - s_off, s_fence};          // part in front survives
    if (s_end > end) it = a.fence_seg.emplace(end, Runtime::Arena::Seg{s_end - end, s_fence}).first;  // part behind
  }
  auto mine = a.fence_seg.emplace(off, Runtime::Arena::Seg{len, fence}).first;
  // fold equal neighbours together so the map stays as small as the arena's block structure
  auto next = std::next(mine);
  if (next != a.fence_seg.end() && next->second.fence == fence && mine->first + mine->second.len == next->first) {
    mine->second.len += next->second.len;
    a.fence_seg.erase(next);
  }
  if (mine != a.fence_seg.begin()) {
    auto prev = std::prev(mine);
    if (prev->second.fence == fence && prev->first + prev->second.len == mine->first) {
      prev->second.len += mine->second.len;
      a.fence_seg.erase(mine);
    }
  }
}

// Latest fence among the segments that [off, off + len) overlaps.
uint64_t arena_fence_of(const Runtime::Arena &a, size_t off, size_t len) {
  uint64_t fence = Runtime::kNoFence;
  auto it = a.fence_seg.upper_bound(off);
  if (it != a.fence_seg.begin()) --it;
  for (; it != a.fence_seg.end() && it->first < off + len; ++it)
    if (it->first + it->second.len > off) fence = later_fence(fence, it->second.fence);
  return fence;
}

void *arena_alloc(Runtime::Arena &a, size_t want, uint64_t *fence) {
  auto it = a.free_by_len.lower_bound(want);  // best fit
  if (it == a.free_by_len.end()) return nullptr;
  const size_t len = it->first, off = it->second;
  *fence = arena_fence_of(a, off, want);
  arena_erase_free(a, off, len);
  if (len > want) arena_insert_free(a, off + want, len - want);
  void *ptr = a.base + off;
  a.used[ptr] = want;
  a.used_bytes += want;
  return ptr;
}

// Returns false when `ptr` does not belong to the arena.  `fence` is the release
// fence of the block.
bool arena_free(Runtime::Arena &a, void *ptr, uint64_t fence) {
  auto it = a.used.find(ptr);
  if (it == a.used.end()) return false;
  size_t off = (size_t)((char *)ptr - a.base), len = it->second;
  a.used_bytes -= len;
  a.used.erase(it);
  arena_set_fence(a, off, len, fence);
  auto next = a.free_by_off.lower_bound(off);
  if (next != a.free_by_off.end() && next->first == off + len) {  // merge with the range behind
    const size_t nlen = next->second;
    arena_erase_free(a, next->first, nlen);
    len += nlen;
  }
  auto prev = a.free_by_off.lower_bound(off);
  if (prev != a.free_by_off.begin()) {
    --prev;
    if (prev->first + prev->second == off) {  // merge with the range in front
      const size_t poff = prev->first, plen = prev->second;
      arena_erase_free(a, poff, plen);
      off = poff;
      len += plen;
    }
  }
  arena_insert_free(a, off, len);
  if (a.retired && a.used.empty()) {
    (void)hipFree(a.base);
    a = Runtime::Arena();
  }
  return true;
}

void *pool_alloc(Runtime::Pool &p, size_t bytes, bool device, size_t limit) {
  const size_t want = round_size(bytes);
  void *ptr = nullptr;
  auto it = p.free_blocks.lower_bound(want);
  // accept a cached block when it wastes at most 1/8 of its size
  if (it != p.free_blocks.end() && it->first - want <= it->first / 8) {
    ptr = it->second;
    p.free_blocks.erase(it);
  }
  for (int attempt = 0; !ptr && attempt < 2; ++attempt) {
    if (limit == 0 || p.reserved + want <= limit) {
      hipError_t e = device ? hipMalloc(&ptr, want) : hipHostMalloc(&ptr, want, hipHostMallocDefault);
      if (e == hipSuccess && ptr) {
        p.block_size[ptr] = want;
        p.reserved += want;
        break;
      }
      ptr = nullptr;
      (void)hipGetLastError();  // clear the sticky out-of-memory error
    }
    if (attempt == 0) {
      if (p.free_blocks.empty()) break;
      release_cached(p, device, want, limit);
    }
  }
  if (ptr) {
    p.in_use += p.block_size[ptr];
    const size_t total = p.in_use + (device ? rt().arena.used_bytes : 0);
    if (total > p.peak_in_use) p.peak_in_use = total;
  }
  return ptr;
}

void pool_free(Runtime::Pool &p, void *ptr) {
  if (!ptr) return;
  auto it = p.block_size.find(ptr);
  if (it == p.block_size.end()) return;  // not ours (e.g. a borrowed numpy buffer)
  p.free_blocks.emplace(it->second, ptr);
  p.in_use -= it->second;
}

}  // namespace

// Creates the arena for the current budget: everything the budget leaves after the
// blocks already handed out by the pool.  Called with the lock held.
void arena_open(Runtime &r) {
  release_cached(r.dev, true, 0, 0);  // nothing stays cached outside the arena
  if (r.dev_limit <= r.dev.in_use) return;
  const size_t size = (r.dev_limit - r.dev.in_use) / 65536 * 65536;
  if (size == 0) return;
  void *base = nullptr;
  if (hipMalloc(&base, size) != hipSuccess || !base) {
    (void)hipGetLastError();
    return;  // not enough physical memory for the budget: the pool path enforces it instead
  }
  r.arena.base = (char *)base;
  r.arena.size = size;
  arena_insert_free(r.arena, 0, size);
  r.arena.fence_seg[0] = {size, Runtime::kNoFence};
}

// Records a release fence on the one stream that runs kernels and returns its
// number; kConservative when there is no such single stream (none yet, or several).
// Called with the lock held.
uint64_t record_release_fence(Runtime &r) {
  hipStream_t only = nullptr;
  int kernel_streams = 0;
  for (auto &rec : r.streams)
    if (rec.runs_kernels) {
      only = rec.stream;
      ++kernel_streams;
    }
  if (kernel_streams != 1) return Runtime::kConservative;
  const uint64_t number = r.fence_count + 1;
  hipEvent_t &ev = r.fence_ring[number % Runtime::kFenceRing];
  if (!ev && hipEventCreateWithFlags(&ev, hipEventDisableTiming) != hipSuccess) {
    ev = nullptr;
    (void)hipGetLastError();
    return Runtime::kConservative;
  }
  if (hipEventRecord(ev, only) != hipSuccess) {
    (void)hipGetLastError();
    return Runtime::kConservative;
  }
  r.fence_count = number;
  return number;
}

size_t block_bytes(size_t bytes) { return round_size(bytes); }

int drop_all_kept();  // below, with the registry of kept blocks
static void *device_alloc_once(size_t bytes);
// Blocks kept for a later call (keep_set) are a convenience, never a reason to fail:
// when the device has no room, they are given back and the request is tried again.
void *device_alloc(size_t bytes) {
  void *p = device_alloc_once(bytes);
  if (!p && drop_all_kept() > 0) p = device_alloc_once(bytes);
  return p;
}
static void *device_alloc_once(size_t bytes) {
  Runtime &r = rt();
  std::lock_guard<std::mutex> g(r.mu);
  r.init();
  if (r.dev_limit != 0) {
    if (!r.arena.base) arena_open(r);
    if (r.arena.base && !r.arena.retired) {
      uint64_t fence = Runtime::kNoFence;
      void *ptr = arena_alloc(r.arena, round_size(bytes), &fence);
      if (ptr) {
        r.block_fence[ptr] = fence;
        const size_t total = r.dev.in_use + r.arena.used_bytes;
        if (total > r.dev.peak_in_use) r.dev.peak_in_use = total;
      }
      return ptr;
    }
  }
  // blocks still alive in an arena that an earlier budget left behind count against this one
  size_t limit = r.dev_limit;
  if (limit != 0 && r.arena.base) limit = limit > r.arena.used_bytes ? limit - r.arena.used_bytes : 1;
  void *ptr = pool_alloc(r.dev, bytes, true, limit);
  if (ptr) {
    auto it = r.pool_fence.find(ptr);
    r.block_fence[ptr] = it == r.pool_fence.end() ? Runtime::kNoFence : it->second;
  }
  return ptr;
}
void device_free(void *p) {
  if (!p) return;
  Runtime &r = rt();
  std::lock_guard<std::mutex> g(r.mu);
  if (r.block_fence.erase(p) == 0) return;  // not a block handed out by device_alloc
  // the next fence to be recorded covers this release (an event per release would put
  // a marker into the compute stream each time: measured 0.75 ms per ResNet-50 step)
  const uint64_t fence = r.fence_count + 1;
  if (r.arena.base && arena_free(r.arena, p, fence)) return;
  r.pool_fence[p] = fence;
  pool_free(r.dev, p);
  // a pool block returned while a budget is active must not linger in the cache
  if (r.dev_limit != 0 && r.arena.base) release_cached(r.dev, true, 0, 0);
}

// Makes `s` wait until the previous life of the storage behind `ptr` (a block handed
// out by device_alloc and not used since) is over.  Returns 0, or 1 when no fence
// is known and the caller has to wait for all kernel streams instead.
int wait_for_previous_life(void *ptr, hipStream_t s) {
  Runtime &r = rt();
  std::lock_guard<std::mutex> g(r.mu);
  auto it = r.block_fence.find(ptr);
  if (it == r.block_fence.end() || it->second > r.fence_count) return 1;  // unknown, or its fence was never recorded
  if (it->second == Runtime::kNoFence) return 0;
  // a slot reused since then holds a later fence of the same stream
  hipEvent_t ev = r.fence_ring[it->second % Runtime::kFenceRing];
  if (!ev || hipStreamWaitEvent(s, ev, 0) != hipSuccess) {
    (void)hipGetLastError();
    return 1;
  }
  return 0;
}
void *pinned_alloc(size_t bytes) {
  Runtime &r = rt();
  std::lock_guard<std::mutex> g(r.mu);
  r.init();
  return pool_alloc(r.host, bytes, false, 0);
}
void pinned_free(void *p) {
  Runtime &r = rt();
  std::lock_guard<std::mutex> g(r.mu);
  pool_free(r.host, p);
}

// Stream an op launches on.  Marks the stream as one that runs kernels, so that
// copies on other streams know to order themselves behind it.
hipStream_t stream_of(void **cell) {
  if (!cell) return nullptr;
  hipStream_t s = reinterpret_cast<hipStream_t>(*cell);
  Runtime &r = rt();
  std::lock_guard<std::mutex> g(r.mu);
  for (auto &rec : r.streams)
    if (rec.stream == s) {
      rec.runs_kernels = true;
      break;
    }
  return s;
}

// Ticket counters for the contraction kernels that fold k-split tiles in the kernel
// itself: kFoldTicketSlots words per stream, zero between launches (the kernels
// restore the zeros; launches on one stream run one after the other, so they can
// share the words).  Allocated on first use and cleared by a fill kernel on `s`.
// Streams made by DLGpuCreatecudaStream keep their words in their record (released
// with the stream); any other handle -- the null stream, a caller's own stream -- gets
// words of its own under its handle, so two such streams never count on the same words.
unsigned *fold_tickets(hipStream_t s) {
  Runtime &r = rt();
  auto cell_of = [&]() -> unsigned ** {  // with r.mu held
    static std::unordered_map<hipStream_t, unsigned *> foreign_stream_tickets;
    for (auto &rec : r.streams)
      if (rec.stream == s) return &rec.fold_tickets;
    return &foreign_stream_tickets[s];
  };
  {
    std::lock_guard<std::mutex> g(r.mu);
    if (unsigned *have = *cell_of()) return have;
  }
  // first use on this stream: 16 KiB straight from the device (not the pool: the words
  // live as long as the stream).  When the device is full, the kept by-products go first.
  void *p = nullptr;
  if (hipMalloc(&p, kFoldTicketSlots * sizeof(unsigned)) != hipSuccess || !p) {
    (void)hipGetLastError();
    p = nullptr;
    if (drop_all_kept() == 0 || hipMalloc(&p, kFoldTicketSlots * sizeof(unsigned)) != hipSuccess || !p) {
      (void)hipGetLastError();
      return nullptr;
    }
  }
  hipLaunchKernelGGL(zero_words_kernel, dim3(cdiv(kFoldTicketSlots, 256)), dim3(256), 0, s, (unsigned *)p,
                     kFoldTicketSlots);
  std::lock_guard<std::mutex> g(r.mu);
  unsigned **cell = cell_of();
  if (*cell) {  // another thread got there first on the same stream
    (void)hipFree(p);
    return *cell;
  }
  *cell = (unsigned *)p;
  return *cell;
}

// Stream for the entry points that have no stream argument (the reference runs
// them on the legacy default stream, which is ordered against every other stream).
// When exactly one stream created here has run kernels, work placed on it is ordered
// the same way with respect to everything this library enqueues -- behind that
// stream's earlier kernels, in front of its later ones, and copies on other streams
// order themselves against it -- without the default stream's wait for all streams,
// which stalls the host once per call.  Otherwise: the default stream.
hipStream_t streamless_launch_stream() {
  Runtime &r = rt();
  std::lock_guard<std::mutex> g(r.mu);
  hipStream_t only = nullptr;
  int kernel_streams = 0;
  for (auto &rec : r.streams)
    if (rec.runs_kernels) {
      only = rec.stream;
      ++kernel_streams;
    }
  return kernel_streams == 1 ? only : nullptr;
}

bool sync_every_op() {
  Runtime &r = rt();
  std::lock_guard<std::mutex> g(r.mu);
  r.init();
  return r.sync_ops;
}

int finish(hipStream_t s, const char *what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    fprintf(stderr, "[tinyflow_amd] %s: launch failed: %s\n", what, hipGetErrorString(e));
    return -1;
  }
  if (sync_every_op()) {
    e = hipStreamSynchronize(s);
    if (e != hipSuccess) {
      fprintf(stderr, "[tinyflow_amd] %s: %s\n", what, hipGetErrorString(e));
      return -1;
    }
  }
  return 0;
}

int num_cus() {
  Runtime &r = rt();
  std::lock_guard<std::mutex> g(r.mu);
  if (r.cus == 0) {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) == hipSuccess &&
        hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0)
      r.cus = n;
    else
      r.cus = 256;
  }
  return r.cus;
}

}  // namespace tf

using namespace tf;

// ------------------------------------------------------------------ arrays

static size_t array_bytes(const DLArray *a) { return (size_t)numel(a) * sizeof(float); }

extern "C" int DLArrayAlloc(const index_t *shape, index_t ndim_in, DLContext ctx,
                            DLArrayHandle *out, int *memorytoSaving) {
  // The binding passes ndim as a 32-bit c_int although the prototype says int64:
  // only the low word is defined.
  const int ndim = (int)(ndim_in & 0xffffffff);
  TF_REQUIRE(shape && out && ndim >= 0 && ndim <= 8, "bad arguments (ndim=%d)", ndim);
  TF_REQUIRE(ctx.device_type == kCPU || ctx.device_type == kGPU, "unknown device type %d",
             (int)ctx.device_type);
  size_t bytes = sizeof(float);
  for (int i = 0; i < ndim; ++i) {
    TF_REQUIRE(shape[i] >= 0, "negative extent");
    TF_REQUIRE(shape[i] == 0 || bytes <= ((size_t)1 << 62) / (size_t)shape[i], "shape overflows the address space");
    bytes *= (size_t)shape[i];
  }
  void *data = nullptr;
  if (ctx.device_type == kGPU) {
    TF_HIP(hipSetDevice(ctx.device_id));
    data = device_alloc(bytes);
  } else {
    data = pinned_alloc(bytes);
  }
  if (!data) {
    // out-of-memory convention of the reference: report the size, leave *out alone
    if (memorytoSaving) *memorytoSaving = shortfall(bytes);
    return 0;
  }
  DLArray *arr = new DLArray();
  arr->data = data;
  arr->ctx = ctx;
  arr->ndim = ndim;
  arr->shape = new int64_t[ndim > 0 ? ndim : 1];
  for (int i = 0; i < ndim; ++i) arr->shape[i] = shape[i];
  *out = arr;
  return 0;
}

// ---- by-products kept across calls ---------------------------------------------------
namespace {
struct Kept {
  const char *lo, *hi;  // bytes of the source array
  void **slot;          // the owner's pointer to the kept block; cleared when the block is dropped
  size_t block_bytes;   // size of the kept block
  hipStream_t stream;   // stream whose work produced the block: only a call on it may take it
  int tag;              // what the block is (the owner's code for form and tile)
};
std::mutex kept_mu;
std::vector<Kept> kept;
std::atomic<int> kept_count{0};
std::atomic<long long> kept_total{0}, taken_total{0};  // blocks registered / handed to a later call
size_t kept_bytes = 0;                                 // with kept_mu held: bytes of all kept blocks

// All kept blocks together may hold at most an eighth of the device's memory (36 GB of
// 288): the five benchmark configurations keep 1 - 4 GB, so this only bounds a
// pathological graph (many large Winograd layers whose backward never runs).
size_t kept_cap() {
  static const size_t cap = [] {
    size_t free_b = 0, total_b = 0;
    if (hipMemGetInfo(&free_b, &total_b) != hipSuccess) {
      (void)hipGetLastError();
      return (size_t)4 << 30;
    }
    return total_b / 8;
  }();
  return cap;
}

// with kept_mu held
void drop_at(size_t i) {
  if (*kept[i].slot) device_free(*kept[i].slot);
  *kept[i].slot = nullptr;
  kept_bytes -= kept[i].block_bytes;
  kept[i] = kept.back();
  kept.pop_back();
  kept_count.store((int)kept.size(), std::memory_order_release);
}
}  // namespace

namespace tf {

bool keep_has_room(size_t block_bytes) {
  const size_t cap = kept_cap();
  std::lock_guard<std::mutex> g(kept_mu);
  return kept_bytes + block_bytes <= cap;
}

void keep_set(void **slot, void *block, size_t block_bytes, const void *src, size_t src_bytes, hipStream_t stream,
              int tag) {
  std::lock_guard<std::mutex> g(kept_mu);
  for (size_t i = 0; i < kept.size(); ++i)
    if (kept[i].slot == slot) {
      drop_at(i);
      break;
    }
  *slot = block;
  kept_total.fetch_add(1, std::memory_order_relaxed);
  kept.push_back({(const char *)src, (const char *)src + src_bytes, slot, block_bytes, stream, tag});
  kept_bytes += block_bytes;
  kept_count.store((int)kept.size(), std::memory_order_release);
}

void *keep_take(void **slot, const void *src, hipStream_t stream, int tag) {
  if (kept_count.load(std::memory_order_acquire) == 0) return nullptr;
  std::lock_guard<std::mutex> g(kept_mu);
  for (size_t i = 0; i < kept.size(); ++i)
    if (kept[i].slot == slot) {
      if (kept[i].lo != (const char *)src || kept[i].stream != stream || kept[i].tag != tag) return nullptr;
      void *block = *slot;
      *slot = nullptr;
      drop_at(i);
      taken_total.fetch_add(1, std::memory_order_relaxed);
      return block;
    }
  return nullptr;
}

void note_write(const void *ptr, size_t bytes) {
  if (kept_count.load(std::memory_order_acquire) == 0) return;
  const char *lo = (const char *)ptr, *hi = lo + bytes;
  std::lock_guard<std::mutex> g(kept_mu);
  for (size_t i = 0; i < kept.size();)
    if (lo < kept[i].hi && kept[i].lo < hi) drop_at(i);
    else ++i;
}

void note_write_everything() { (void)drop_all_kept(); }

int drop_all_kept() {
  if (kept_count.load(std::memory_order_acquire) == 0) return 0;
  std::lock_guard<std::mutex> g(kept_mu);
  const int n = (int)kept.size();
  while (!kept.empty()) drop_at(kept.size() - 1);
  return n;
}

bool device_budget_active() {
  Runtime &r = rt();
  std::lock_guard<std::mutex> g(r.mu);
  return r.dev_limit != 0;
}

}  // namespace tf

extern "C" int DLGpuKeptByproductCounts(long long *kept_blocks, long long *taken_blocks, int *held_now) {
  if (kept_blocks) *kept_blocks = kept_total.load(std::memory_order_relaxed);
  if (taken_blocks) *taken_blocks = taken_total.load(std::memory_order_relaxed);
  if (held_now) *held_now = kept_count.load(std::memory_order_acquire);
  return 0;
}

extern "C" int DLArrayFree(DLArrayHandle handle) {
  announce_write(handle);
  if (!handle) return 0;
  if (handle->data) {
    if (handle->ctx.device_type == kGPU) device_free(handle->data);
    else pinned_free(handle->data);
  }
  delete[] handle->shape;
  delete handle;
  return 0;
}

namespace {

hipMemcpyKind copy_kind(const DLArray *from, const DLArray *to) {
  const bool fg = from->ctx.device_type == kGPU, tg = to->ctx.device_type == kGPU;
  if (fg && tg) return hipMemcpyDeviceToDevice;
  if (fg) return hipMemcpyDeviceToHost;
  if (tg) return hipMemcpyHostToDevice;
  return hipMemcpyHostToHost;
}

// Make `s` wait for everything already enqueued on the other kernel-running
// streams created through DLGpuCreatecudaStream: whatever produced the source, or
// still reads the destination's recycled storage, was launched on one of them.
// Copy-only streams are skipped, so an offload and a prefetch stream stay
// independent of each other.
int wait_for_other_streams(hipStream_t s) {
  Runtime &r = rt();
  std::lock_guard<std::mutex> g(r.mu);
  for (auto &rec : r.streams) {
    if (rec.stream == s || !rec.runs_kernels) continue;
    TF_HIP(hipEventRecord(rec.event, rec.stream));
    TF_HIP(hipStreamWaitEvent(s, rec.event, 0));
  }
  return 0;
}

// True when an op entry point has launched on `s`: later kernels of the step are
// then enqueued behind whatever is put on `s` now.
bool stream_runs_kernels(hipStream_t s) {
  Runtime &r = rt();
  std::lock_guard<std::mutex> g(r.mu);
  for (auto &rec : r.streams)
    if (rec.stream == s) return rec.runs_kernels;
  return false;
}

}  // namespace

// Decision table of the streamed copy, exported for the host-logic test: does
// DLArrayCopyFromTo wait for the copy before it returns?  kind: 0 host->device,
// 1 device->host, 2 device->device.
extern "C" int DLArrayCopyWaitsForCompletion(int kind, int stream_runs_kernels_flag, int sync_every_op_flag) {
  if (kind != 2) return 1;                  // host memory must be readable / reusable on return
  if (sync_every_op_flag) return 1;
  return stream_runs_kernels_flag ? 0 : 1;  // a copy-only stream orders nothing behind the copy
}

extern "C" int DLArrayCopyFromTo(DLArrayHandle from, DLArrayHandle to, DLStreamHandle stream) {
  announce_write(to);
  TF_REQUIRE(from && to && from->data && to->data, "null array");
  const size_t bytes = array_bytes(from);
  TF_REQUIRE(bytes == array_bytes(to), "size mismatch (%zu vs %zu bytes)", bytes, array_bytes(to));
  const hipMemcpyKind kind = copy_kind(from, to);
  if (bytes == 0) return 0;
  if (kind == hipMemcpyHostToHost) {
    memcpy(to->data, from->data, bytes);
    return 0;
  }
  if (stream == nullptr) {
    // synchronous form: everything enqueued so far is finished first, so the
    // caller sees the results of all preceding ops
    TF_HIP(hipDeviceSynchronize());
    TF_HIP(hipMemcpy(to->data, from->data, bytes, kind));
    if (kind == hipMemcpyDeviceToDevice) TF_HIP(hipDeviceSynchronize());
    return 0;
  }
  hipStream_t s = reinterpret_cast<hipStream_t>(*reinterpret_cast<void **>(stream));
  if (wait_for_other_streams(s) != 0) return -1;
  TF_HIP(hipMemcpyAsync(to->data, from->data, bytes, kind, s));
  // Host memory must be readable / reusable on return.  A device-to-device copy on
  // the stream the kernels run on is only ever observed by later work of that
  // stream, so it stays asynchronous; on any other stream nothing would order the
  // readers of `to` (or a reuse of `from`'s storage after DLArrayFree) behind the
  // copy, so the call waits for it as the reference does (src/c_runtime_api.cc:148-158).
  const int kind_code = kind == hipMemcpyHostToDevice ? 0 : kind == hipMemcpyDeviceToHost ? 1 : 2;
  if (DLArrayCopyWaitsForCompletion(kind_code, stream_runs_kernels(s) ? 1 : 0, sync_every_op() ? 1 : 0))
    TF_HIP(hipStreamSynchronize(s));
  return 0;
}

// Records, now, the fence that covers the last release of this array's storage
// (no counterpart in the reference).  Called right after DLArrayAlloc by whoever
// will later fill the array with DLArrayCopyIntoFresh: the copy then waits for the
// work that was enqueued up to this call at most, not up to the copy.
extern "C" int DLArrayPrepareFresh(DLArrayHandle arr) {
  announce_write(arr);
  TF_REQUIRE(arr && arr->data && arr->ctx.device_type == kGPU, "not a device array");
  Runtime &r = rt();
  std::lock_guard<std::mutex> g(r.mu);
  auto it = r.block_fence.find(arr->data);
  TF_REQUIRE(it != r.block_fence.end(), "not an array from DLArrayAlloc");
  if (it->second == r.fence_count + 1 && record_release_fence(r) == Runtime::kConservative)
    it->second = Runtime::kConservative;
  return 0;
}

// Host -> device copy into an array that came from DLArrayAlloc and has not been
// used since (no counterpart in the reference; the prefetch of the swap path).
// DLArrayCopyFromTo must assume that kernels already enqueued may still read the
// destination and therefore waits for all of them; here only the previous life of
// the destination's storage has to be over, which is known from the fence recorded
// after that storage was released (see DLArrayPrepareFresh; without that call the
// copy waits for everything enqueued, like DLArrayCopyFromTo) -- so the copy overlaps
// with whatever the compute stream is doing.  Returns after the copy has completed.
extern "C" int DLArrayCopyIntoFresh(DLArrayHandle from, DLArrayHandle to, DLStreamHandle stream) {
  announce_write(to);
  TF_REQUIRE(from && to && from->data && to->data && stream, "null argument");
  TF_REQUIRE(from->ctx.device_type == kCPU && to->ctx.device_type == kGPU, "host to device only");
  const size_t bytes = array_bytes(from);
  TF_REQUIRE(bytes == array_bytes(to), "size mismatch (%zu vs %zu bytes)", bytes, array_bytes(to));
  if (bytes == 0) return 0;
  hipStream_t s = reinterpret_cast<hipStream_t>(*reinterpret_cast<void **>(stream));
  if (wait_for_previous_life(to->data, s) != 0 && wait_for_other_streams(s) != 0) return -1;
  TF_HIP(hipMemcpyAsync(to->data, from->data, bytes, hipMemcpyHostToDevice, s));
  TF_HIP(hipStreamSynchronize(s));
  return 0;
}

extern "C" int getInt(int *intp) { return intp ? *intp : 0; }

// Device-memory budget of the allocator (no counterpart in the reference, which
// is bounded by the physical card): bytes <= 0 removes the limit.  Cached blocks
// are given back until the budget holds; arrays in use are not touched.
extern "C" int DLGpuSetDeviceMemoryLimit(int64_t bytes) {
  note_write_everything();  // nothing is kept from call to call under a budget
  Runtime &r = rt();
  std::lock_guard<std::mutex> g(r.mu);
  r.init();
  r.dev_limit = bytes > 0 ? (size_t)bytes : 0;
  // the arena was sized for the previous budget: retire it (it is handed back
  // when its last block is freed) and let the next allocation open a new one
  if (r.arena.base) {
    if (r.arena.used.empty()) {
      (void)hipFree(r.arena.base);
      r.arena = Runtime::Arena();
    } else {
      r.arena.retired = true;
    }
  }
  if (r.dev_limit) release_cached(r.dev, true, 0, r.dev_limit);
  return 0;
}

// Bytes held from HIP (in use + cached), bytes in use, and the high-water mark of
// bytes in use since the last call with reset_peak != 0 (no reference counterpart).
extern "C" int DLGpuGetDeviceMemoryStats(int64_t *reserved, int64_t *in_use, int64_t *peak_in_use,
                                         int reset_peak) {
  Runtime &r = rt();
  std::lock_guard<std::mutex> g(r.mu);
  if (reserved) *reserved = (int64_t)(r.dev.reserved + r.arena.size);
  if (in_use) *in_use = (int64_t)(r.dev.in_use + r.arena.used_bytes);
  if (peak_in_use) *peak_in_use = (int64_t)r.dev.peak_in_use;
  if (reset_peak) r.dev.peak_in_use = r.dev.in_use + r.arena.used_bytes;
  return 0;
}

// ----------------------------------------------------- streams and handles

extern "C" int DLGpuCreatecudaStream(void **cell) {
  TF_REQUIRE(cell, "null cell");
  hipStream_t s = nullptr;
  // default priority, blocking with respect to the legacy default stream: the
  // stream-less entry points (DLGpuRelu, DLGpuReluGradient) launch on the
  // default stream and are ordered against every stream created here.
  TF_HIP(hipStreamCreateWithFlags(&s, hipStreamDefault));
  hipEvent_t ev = nullptr;
  TF_HIP(hipEventCreateWithFlags(&ev, hipEventDisableTiming));
  {
    Runtime &r = rt();
    std::lock_guard<std::mutex> g(r.mu);
    r.init();
    r.streams.push_back({s, ev, false, nullptr});
  }
  *cell = s;
  return 0;
}

extern "C" int DLGpuDestroycudaStream(void **cell) {
  TF_REQUIRE(cell, "null cell");
  note_write_everything();  // kept blocks are ordered by the stream that made them
  hipStream_t s = reinterpret_cast<hipStream_t>(*cell);
  hipEvent_t ev = nullptr;
  bool found = false;
  {
    Runtime &r = rt();
    std::lock_guard<std::mutex> g(r.mu);
    for (size_t i = 0; i < r.streams.size(); ++i)
      if (r.streams[i].stream == s) {
        ev = r.streams[i].event;
        if (r.streams[i].fold_tickets) (void)hipFree(r.streams[i].fold_tickets);  // waits for the device
        r.streams.erase(r.streams.begin() + i);
        found = true;
        break;
      }
  }
  TF_REQUIRE(found, "not a stream created by DLGpuCreatecudaStream");
  TF_HIP(hipStreamSynchronize(s));
  TF_HIP(hipEventDestroy(ev));
  TF_HIP(hipStreamDestroy(s));
  *cell = nullptr;
  return 0;
}

static int make_handle(void **cell, void **stream_cell) {
  TF_REQUIRE(cell, "null cell");
  Handle *h = new Handle();
  h->magic = kMagicHandle;
  h->stream = stream_of(stream_cell);
  *cell = h;
  return 0;
}
static int drop_handle(void **cell) {
  TF_REQUIRE(cell && *cell, "null handle");
  Handle *h = reinterpret_cast<Handle *>(*cell);
  TF_REQUIRE(h->magic == kMagicHandle, "not a handle created by this library");
  h->magic = 0;
  delete h;
  *cell = nullptr;
  return 0;
}

extern "C" int DLGpuCreatecudnnHandle(void **handle, void **stream) { return make_handle(handle, stream); }
extern "C" int DLGpuDestroycudnnHandle(void **handle) { return drop_handle(handle); }
extern "C" int DLGpuCreatecublasHandle(void **handle, void **stream) { return make_handle(handle, stream); }
extern "C" int DLGpuDestroycublasHandle(void **handle) { return drop_handle(handle); }

// ---------------------------------------------------------------- testPcie

// Host<->device bandwidth probe: 16 MiB each way, pageable and pinned, with a
// byte-exact round-trip check (reference: src/gpu_op.cu:4915-5005).
extern "C" int testPcie() {
  const size_t bytes = (size_t)16 << 20;
  const size_t n = bytes / sizeof(float);
  float *pageable_a = (float *)malloc(bytes), *pageable_b = (float *)malloc(bytes);
  float *pinned_a = nullptr, *pinned_b = nullptr, *dev = nullptr;
  TF_REQUIRE(pageable_a && pageable_b, "host malloc failed");
  TF_HIP(hipHostMalloc((void **)&pinned_a, bytes, hipHostMallocDefault));
  TF_HIP(hipHostMalloc((void **)&pinned_b, bytes, hipHostMallocDefault));
  TF_HIP(hipMalloc((void **)&dev, bytes));
  for (size_t i = 0; i < n; ++i) pageable_a[i] = pinned_a[i] = (float)i;
  hipEvent_t t0, t1;
  TF_HIP(hipEventCreate(&t0));
  TF_HIP(hipEventCreate(&t1));
  struct Case { const char *name; float *src, *dst; } cases[2] = {
      {"pageable", pageable_a, pageable_b}, {"pinned", pinned_a, pinned_b}};
  int rc = 0;
  for (auto &c : cases) {
    float ms = 0.f;
    memset(c.dst, 0, bytes);
    TF_HIP(hipEventRecord(t0, nullptr));
    TF_HIP(hipMemcpy(dev, c.src, bytes, hipMemcpyHostToDevice));
    TF_HIP(hipEventRecord(t1, nullptr));
    TF_HIP(hipEventSynchronize(t1));
    TF_HIP(hipEventElapsedTime(&ms, t0, t1));
    printf("%s host->device: %.2f GB/s\n", c.name, bytes * 1e-6 / ms);
    TF_HIP(hipEventRecord(t0, nullptr));
    TF_HIP(hipMemcpy(c.dst, dev, bytes, hipMemcpyDeviceToHost));
    TF_HIP(hipEventRecord(t1, nullptr));
    TF_HIP(hipEventSynchronize(t1));
    TF_HIP(hipEventElapsedTime(&ms, t0, t1));
    printf("%s device->host: %.2f GB/s\n", c.name, bytes * 1e-6 / ms);
    if (memcmp(c.src, c.dst, bytes) != 0) {
      printf("%s round trip MISMATCH\n", c.name);
      rc = -1;
    }
  }
  (void)hipEventDestroy(t0);
  (void)hipEventDestroy(t1);
  (void)hipFree(dev);
  (void)hipHostFree(pinned_a);
  (void)hipHostFree(pinned_b);
  free(pageable_a);
  free(pageable_b);
  return rc;
}
