// Internal helpers shared by the HIP sources of libc_runtime_api.so.
// Nothing here is part of the C-ABI; the exported surface is include/c_runtime_api.h.
#pragma once

#include <hip/hip_runtime.h>
#include <cstdint>
#include <cstdio>
#include <cstdlib>

#include "c_runtime_api.h"

namespace tf {

// ---- device scratch / array storage: caching allocator (runtime.hip) -------
// Blocks are recycled by size; a freed block may still be read by kernels that
// are already enqueued, which is safe because every consumer is ordered after
// them (same stream, or cross-stream wait inserted by DLArrayCopyFromTo).
void *device_alloc(size_t bytes);  // nullptr when the device (or the cap) is exhausted
void device_free(void *p);
size_t block_bytes(size_t bytes);  // what a block of that many bytes occupies (the allocator's rounding)
void *pinned_alloc(size_t bytes);
void pinned_free(void *p);

// ---- streams ----------------------------------------------------------------
hipStream_t stream_of(void **cell);      // cell written by DLGpuCreatecudaStream; NULL -> default stream
hipStream_t streamless_launch_stream();  // for entry points without a stream argument
bool sync_every_op();                    // TINYFLOW_SYNC_EVERY_OP=1
int finish(hipStream_t s, const char *what);  // launch-error check (+ optional sync)

// Zeroed counters for the in-kernel fold of the contraction kernels, one set per stream.
constexpr int kFoldTicketSlots = 4096;
unsigned *fold_tickets(hipStream_t s);

// ---- small host utilities -----------------------------------------------------
inline int64_t numel(const DLArray *a) {
  int64_t n = 1;
  for (int i = 0; i < a->ndim; ++i) n *= a->shape[i];
  return n;
}
inline bool same_shape(const DLArray *a, const DLArray *b) {
  if (a->ndim != b->ndim) return false;
  for (int i = 0; i < a->ndim; ++i)
    if (a->shape[i] != b->shape[i]) return false;
  return true;
}
inline bool on_gpu(const DLArray *a) { return a && a->data && a->ctx.device_type == kGPU; }

inline int cdiv(int64_t a, int64_t b) { return (int)((a + b - 1) / b); }

// Value stored through `memorytoSaving` when an allocation of `bytes` fails.  The
// caller reads "non-zero" as "out of memory, this much was wanted"
// (src/c_runtime_api.cc:109-113 casts the size to int); the cast is saturated here
// so that a request of 2 GiB or more can neither wrap to zero nor go negative.
inline int shortfall(size_t bytes) {
  if (bytes == 0) return 1;
  return bytes > (size_t)0x7fffffff ? 0x7fffffff : (int)bytes;
}

// Number of compute units of the current device (256 on MI355X).
int num_cus();

// ---- by-products kept from one call to a later one (runtime.hip) ----------------
// An op may keep a device block that it derived from an input array (the transformed
// input of a Winograd forward call) for a later call on the same input.  Such a block
// is valid only while the input's bytes are unchanged, so every entry point announces
// the arrays it is about to write (or free) before it does anything else, and the
// registry drops what was derived from them.  All device memory behind this ABI is
// written through these entry points, which is what makes the rule complete.
// What a block is (`tag`: the owner's code for form and tile) and the stream whose work
// made it live in the registry entry, under its lock; only a call on that stream asking
// for that tag and that source gets the block.  All kept blocks together are capped at a
// fraction of the device's memory: ask keep_has_room before allocating one.
bool keep_has_room(size_t block_bytes);
void keep_set(void **slot, void *block, size_t block_bytes, const void *src, size_t src_bytes, hipStream_t stream,
              int tag);  // replaces what the slot held
void *keep_take(void **slot, const void *src, hipStream_t stream, int tag);  // the block (caller frees), else null
void note_write(const void *ptr, size_t bytes);
void note_write_everything();
bool device_budget_active();  // a device-memory limit is set: keep nothing
inline void announce_write(const DLArray *a) {
  if (a && a->data && a->ctx.device_type == kGPU) note_write(a->data, (size_t)numel(a) * sizeof(float));
}

}  // namespace tf

#define TF_REQUIRE(cond, ...)                                  \
  do {                                                         \
    if (!(cond)) {                                             \
      fprintf(stderr, "[tinyflow_amd] %s: ", __func__);        \
      fprintf(stderr, __VA_ARGS__);                            \
      fprintf(stderr, "\n");                                   \
      return -1;                                               \
    }                                                          \
  } while (0)

#define TF_HIP(expr)                                                          \
  do {                                                                        \
    hipError_t _e = (expr);                                                   \
    if (_e != hipSuccess) {                                                   \
      fprintf(stderr, "[tinyflow_amd] %s: %s failed: %s\n", __func__, #expr,  \
              hipGetErrorString(_e));                                         \
      return -1;                                                              \
    }                                                                         \
  } while (0)

// Opaque descriptor structs placed behind the `void ***list` arguments.
namespace tf {

constexpr int kMagicConv = 0x74664376;    // 'tfCv'
constexpr int kMagicPool = 0x7466506c;    // 'tfPl'
constexpr int kMagicAct = 0x74664163;     // 'tfAc'
constexpr int kMagicBN = 0x7466424e;      // 'tfBN'
constexpr int kMagicReduce = 0x74665264;  // 'tfRd'
constexpr int kMagicHandle = 0x74664864;  // 'tfHd'

struct Handle {
  int magic;
  hipStream_t stream;
};

struct ConvDesc {
  int magic;
  int N, C, H, W;      // input
  int K, R, S;         // filter (K output channels, C input channels)
  int P, Q;            // output spatial
  int pad_h, pad_w, u, v;
  // Winograd forms: the transformed input V of the last forward call, kept for the
  // grad-filter call of the same step, which needs exactly this array (see keep_set).
  // (the three kept_* pointers are registry slots: written and read only through
  // keep_set / keep_take, which hold the block's tile, form and stream under their lock)
  void *kept_v = nullptr;
  int grad_filter_tile = 0;  // tile of the last grad-filter call that ran in a Winograd form (0: none yet)
  // the same for the transformed filter of grad-data (the filter rotated by 180 degrees),
  // which the forward call's filter transform writes along with its own
  void *kept_u = nullptr;
  int grad_data_tile = 0;    // tile of the last grad-data call that ran in a Winograd form (0: none yet)
  // grad-data and grad-filter both transform dy; whichever runs first writes the other's
  // form along with its own and keeps it (tag kKeptDyForDgrad: grad-data's V, kKeptDyForWgrad: grad-filter's dM)
  void *kept_dy = nullptr;
};
constexpr int kKeptDyForDgrad = 0x100, kKeptDyForWgrad = 0x200;  // or-ed with the tile

struct PoolDesc {
  int magic;
  int N, C, H, W, P, Q;
  int mode;            // 0 max, 1 mean (count includes padding)
  int pad_h, pad_w, u, v, fh, fw;
};

struct ActDesc {
  int magic;
  int mode;
  int64_t n, inner;    // n instances of `inner` = c*h*w elements
  // ReLU only: one bit per element, x > 0, written by the forward call beside y and
  // kept for the backward call of the same step, which then reads dy and the bits
  // (8.125 bytes per element) instead of dy and x (12).  Owned by keep_set / keep_take.
  void *kept_mask = nullptr;
  bool backward_seen = false;   // a forward call keeps bits only once a backward call has used this descriptor
};

struct BNDesc {
  int magic;
  int mode;            // 0 per-activation, 1 spatial
  int N, C, HW;        // x viewed as [N, C, HW]
  int64_t stat_count;  // C*HW (per-activation) or C (spatial)
  // statistics published by the last forward and not yet consumed by a backward
  float *saved_mean, *saved_istd;
};

struct ReduceDesc {
  int magic;
  int ndim;
  int in[5];
  int out[5];
};

template <class T>
inline T *desc_from_list(void ***list, int magic) {
  if (!list || !*list) return nullptr;
  T *d = reinterpret_cast<T *>((*list)[0]);
  if (!d || d->magic != magic) return nullptr;
  return d;
}

}  // namespace tf

// Cross-file kernel launchers.
namespace tf {
// out[i] = sum_s partial[s * count + i] in split order (matmul.hip)
int launch_split_sum(const float *partial, float *out, int64_t count, int splits, hipStream_t s);
int choose_splits(int tiles, int K, int min_k);
// row softmax and its backward over [rows, cols] (reduce.hip)
int launch_softmax_rows(const float *in, float *out, int64_t rows, int cols, hipStream_t s);
int launch_softmax_rows_backward(const float *y, const float *dy, float *dx, int64_t rows, int cols,
                                 hipStream_t s);
}  // namespace tf
