// Host side of the contraction kernels' in-kernel fold (gemm_core.h: Fold): the
// decision which tiles of a launch are folded, and the scratch / ticket buffers.
#pragma once

#include "gemm_core.h"
#include "internal.h"

#include <algorithm>
#include <cstdlib>

namespace tf {
namespace gemm {

// TINYFLOW_FOLD (measurements and tests): 0 no folding, 1 only short k-splits,
// 2 only the remainder round, 3 (default) both.
inline int fold_switch() {
  const char *e = getenv("TINYFLOW_FOLD");
  return e && *e ? atoi(e) : 3;
}

// Measured on the ResNet-50 batch-64 layers: folding in the kernel beats the separate
// sum pass up to five pieces (beyond that one workgroup reading all pieces of its tile
// is slower than the lane-parallel pass), and cutting the remainder round pays when a
// piece still runs at least two reduction stages (a one-stage piece is all prologue)
// of a reduction of at least eight.
constexpr int kMaxFoldedSplits = 5;
constexpr int kMinStagesPerTailPiece = 2;
constexpr int kMinStagesForTail = 8;   // shorter reductions (64 channels) lose more to the extra workgroups than they gain
constexpr int kMaxTailPieces = 8;      // 4, 8 and 16 measured the same

// Rewrites `g` (made by make_geometry for the planned number of k-splits) so that
//   * a split of 2..kMaxFoldedSplits becomes pieces of every tile, folded in the kernel;
//   * an unsplit launch of more than one round over the CUs whose last round is
//     partial folds the tiles of that round: with R leftover tiles each is cut into
//     floor(CUs / R) pieces along the reduction, about one short piece per CU,
//     instead of R whole tiles that keep R CUs busy while the rest idle.
// Depends on the shape and the CU count only, so a layer always gets the same
// summation order.  `tail_ok` = false keeps the remainder round as it is.
inline void plan_fold(Geometry &g, int K, int BK, int batch, bool tail_ok = true) {
  const int mode = fold_switch();
  const int tiles = g.tiles();
  const int k_steps = (K + BK - 1) / BK;
  if (g.splits > 1) {
    if (!(mode & 1) || g.splits > kMaxFoldedSplits || (int64_t)tiles * batch > kFoldTicketSlots) return;
    g.fold_first_tile = 0;
    g.fold_pieces = g.splits;
    g.fold_k_per_piece = g.k_per_split;
    g.splits = 1;
    return;
  }
  if (!(mode & 2) || !tail_ok || batch != 1) return;
  const int cus = num_cus();
  if (tiles <= cus) return;
  const int rest = tiles % cus;
  if (rest == 0) return;
  if (k_steps < kMinStagesForTail) return;
  int pieces = std::min(std::min(cus / rest, k_steps / kMinStagesPerTailPiece), kMaxTailPieces);
  if (pieces < 2) return;
  const int steps_per_piece = (k_steps + pieces - 1) / pieces;
  pieces = (k_steps + steps_per_piece - 1) / steps_per_piece;  // no empty piece
  if (pieces < 2) return;
  g.fold_first_tile = tiles - rest;
  g.fold_pieces = pieces;
  g.fold_k_per_piece = steps_per_piece * BK;
}

struct FoldBuffers {
  float *scratch = nullptr;
  unsigned *tickets = nullptr;
  size_t bytes = 0;
};

// Scratch and tickets for the folded tiles of `g`, entered into `g`: 0 ok (also when
// nothing is folded), 1 when the scratch cannot be had (fb.bytes = size wanted), -1 on error.
inline int acquire_fold(Geometry &g, int bm, int bn, int batch, hipStream_t s, FoldBuffers &fb) {
  if (g.fold_pieces <= 1) return 0;
  fb.bytes = g.fold_scratch_bytes(bm, bn, batch);
  fb.tickets = fold_tickets(s);
  if (!fb.tickets) {
    fprintf(stderr, "[tinyflow_amd] no memory for the fold counters\n");
    return -1;
  }
  fb.scratch = (float *)device_alloc(fb.bytes);
  g.fold_scratch = fb.scratch;
  g.fold_ticket_words = fb.tickets;
  return fb.scratch ? 0 : 1;
}
inline void release_fold(FoldBuffers &fb) {
  if (fb.scratch) device_free(fb.scratch);  // stream-ordered reuse: later users are enqueued behind the kernel
  fb.scratch = nullptr;
}

}  // namespace gemm
}  // namespace tf
