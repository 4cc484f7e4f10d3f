// DLGpuMatrixMultiply: C = op(A) * op(B) on the fp32 MFMA tile engine.
//
// Replaces the cublasSgemm call of the reference (src/gpu_op.cu:1166-1199).
// The same entry point serves the forward product and both gradients the
// autodiff emits for it (dA = dY * B^T, dB = A^T * dY,
// pycode/tinyflow/autodiff.py:477-506), so all four transpose combinations are
// first-class: a transposed operand only changes which loader reads it.
//
// Skinny problems (few output tiles, long reduction - e.g. a batch-32 fully
// connected layer) are split along k into partial products that a second,
// fixed-order pass adds up, so results do not depend on scheduling.
#include "gemm_core.h"
#include "gemm_launch.h"
#include "internal.h"

using namespace tf;
using namespace tf::gemm;

namespace {

// out[i] = sum_s partial[s * count + i], splits added in index order
__global__ __launch_bounds__(256) void split_sum_kernel(const float *__restrict__ partial,
                                                       float *__restrict__ out, int64_t count, int splits) {
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < count; i += stride) {
    float s = partial[i];
    for (int k = 1; k < splits; ++k) s += partial[(int64_t)k * count + i];
    out[i] = s;
  }
}

typedef float f32x4 __attribute__((ext_vector_type(4)));

// Same sum for 16-byte aligned data with count % 4 == 0, with the splits dealt
// round-robin to SG lane groups of a workgroup so that a small output with
// many splits still has enough loads in flight.  Group g adds splits g, g+SG,
// ... in that order, then group 0 adds the SG group sums in index order: the
// order of additions depends on (splits, SG) only, never on timing.
template <int SG>
__global__ __launch_bounds__(256) void split_sum_vec_kernel(const f32x4 *__restrict__ partial,
                                                           f32x4 *__restrict__ out, int64_t count4, int splits) {
  constexpr int COLS = 256 / SG;
  __shared__ f32x4 part[SG][COLS];
  const int col = threadIdx.x % COLS, g = threadIdx.x / COLS;
  const int64_t i = (int64_t)blockIdx.x * COLS + col;
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  if (i < count4) {
    int k = g;
    for (; k + 3 * SG < splits; k += 4 * SG) {
      const f32x4 v0 = __builtin_nontemporal_load(partial + (int64_t)k * count4 + i);
      const f32x4 v1 = __builtin_nontemporal_load(partial + (int64_t)(k + SG) * count4 + i);
      const f32x4 v2 = __builtin_nontemporal_load(partial + (int64_t)(k + 2 * SG) * count4 + i);
      const f32x4 v3 = __builtin_nontemporal_load(partial + (int64_t)(k + 3 * SG) * count4 + i);
      acc = (((acc + v0) + v1) + v2) + v3;
    }
    for (; k < splits; k += SG) acc += __builtin_nontemporal_load(partial + (int64_t)k * count4 + i);
  }
  if (SG == 1) {
    if (i < count4) out[i] = acc;
    return;
  }
  part[g][col] = acc;
  __syncthreads();
  if (g == 0 && i < count4) {
    f32x4 total = part[0][col];
#pragma unroll
    for (int j = 1; j < SG; ++j) total += part[j][col];
    out[i] = total;
  }
}

template <int BM, int BN, int BK, class AL, class BL>
void launch(const AL &al, const BL &bl, const StoreRowMajor &ep, int K, const Geometry &g, hipStream_t s) {
  hipLaunchKernelGGL((gemm_kernel<BM, BN, BK, AL, BL, StoreRowMajor>), dim3(g.blocks()), dim3(THREADS), 0, s,
                     al, bl, ep, K, g.k_per_split, g.tiles_m, g.tiles_n, g.fold());
}

template <int BM, int BN, int BK>
void dispatch(const float *A, bool tA, int lda, uint32_t a_bytes, const float *B, bool tB, int ldb,
              uint32_t b_bytes, const StoreRowMajor &ep, int M, int N, int K, const Geometry &g, hipStream_t s) {
  // 16-byte loads when both operands allow them (alignment, leading dimension and
  // the extent along each operand's contiguous direction multiples of 4)
  const bool vec = vec4_ok(A, lda, tA ? M : K) && vec4_ok(B, ldb, tB ? K : N);
  const FastDiv whole(ONE_SEGMENT);
  if (vec) {
    if (!tA && !tB) {
      Across4<BM, BK> al{A, a_bytes, lda, M, K, whole, 0};
      Along4<BN, BK> bl{B, b_bytes, ldb, N, K, whole, 0};
      launch<BM, BN, BK>(al, bl, ep, K, g, s);
    } else if (tA && !tB) {
      Along4<BM, BK> al{A, a_bytes, lda, M, K, whole, 0};
      Along4<BN, BK> bl{B, b_bytes, ldb, N, K, whole, 0};
      launch<BM, BN, BK>(al, bl, ep, K, g, s);
    } else if (!tA && tB) {
      Across4<BM, BK> al{A, a_bytes, lda, M, K, whole, 0};
      Across4<BN, BK> bl{B, b_bytes, ldb, N, K, whole, 0};
      launch<BM, BN, BK>(al, bl, ep, K, g, s);
    } else {
      Along4<BM, BK> al{A, a_bytes, lda, M, K, whole, 0};
      Across4<BN, BK> bl{B, b_bytes, ldb, N, K, whole, 0};
      launch<BM, BN, BK>(al, bl, ep, K, g, s);
    }
    return;
  }
  if (!tA && !tB) {
    PlainAcross<BM, BK> al{A, a_bytes, lda, M, K};
    PlainAlong<BN, BK> bl{B, b_bytes, ldb, N, K};
    launch<BM, BN, BK>(al, bl, ep, K, g, s);
  } else if (tA && !tB) {
    PlainAlong<BM, BK> al{A, a_bytes, lda, M, K};
    PlainAlong<BN, BK> bl{B, b_bytes, ldb, N, K};
    launch<BM, BN, BK>(al, bl, ep, K, g, s);
  } else if (!tA && tB) {
    PlainAcross<BM, BK> al{A, a_bytes, lda, M, K};
    PlainAcross<BN, BK> bl{B, b_bytes, ldb, N, K};
    launch<BM, BN, BK>(al, bl, ep, K, g, s);
  } else {
    PlainAlong<BM, BK> al{A, a_bytes, lda, M, K};
    PlainAcross<BN, BK> bl{B, b_bytes, ldb, N, K};
    launch<BM, BN, BK>(al, bl, ep, K, g, s);
  }
}

}  // namespace

namespace tf {

int launch_split_sum(const float *partial, float *out, int64_t count, int splits, hipStream_t s) {
  const bool vec = count % 4 == 0 && ((reinterpret_cast<uintptr_t>(partial) | reinterpret_cast<uintptr_t>(out)) & 15u) == 0;
  if (vec) {
    const int64_t count4 = count / 4;
    const f32x4 *p4 = reinterpret_cast<const f32x4 *>(partial);
    f32x4 *o4 = reinterpret_cast<f32x4 *>(out);
    // enough lane groups that about 64 K lanes are busy, as long as each group
    // still has a few splits to add
    int sg = 1;
    while (sg < 16 && count4 * sg < 65536 && splits >= 8 * sg) sg *= 4;
    const unsigned blocks = (unsigned)((count4 + 256 / sg - 1) / (256 / sg));
    if (sg == 1) hipLaunchKernelGGL(split_sum_vec_kernel<1>, dim3(blocks), dim3(256), 0, s, p4, o4, count4, splits);
    else if (sg == 4) hipLaunchKernelGGL(split_sum_vec_kernel<4>, dim3(blocks), dim3(256), 0, s, p4, o4, count4, splits);
    else hipLaunchKernelGGL(split_sum_vec_kernel<16>, dim3(blocks), dim3(256), 0, s, p4, o4, count4, splits);
    return 0;
  }
  int64_t blocks = (count + 255) / 256;
  const int64_t cap = (int64_t)num_cus() * 8;
  if (blocks > cap) blocks = cap;
  if (blocks < 1) blocks = 1;
  hipLaunchKernelGGL(split_sum_kernel, dim3((unsigned)blocks), dim3(256), 0, s, partial, out, count, splits);
  return 0;
}

// Number of k-splits that brings `tiles` output tiles up to about two
// workgroups per CU without making a split shorter than `min_k` reduction steps.
int choose_splits(int tiles, int K, int min_k) {
  const int target = 2 * num_cus();
  if (tiles >= target) return 1;
  int splits = (target + tiles - 1) / tiles;
  const int max_splits = K / min_k;
  if (splits > max_splits) splits = max_splits;
  return splits < 1 ? 1 : splits;
}

}  // namespace tf

extern "C" int DLGpuMatrixMultiply(const DLArrayHandle matA, bool transposeA, const DLArrayHandle matB,
                                   bool transposeB, DLArrayHandle matC, void **handle, void **stream) {
  announce_write(matC);
  (void)handle;
  TF_REQUIRE(on_gpu(matA) && on_gpu(matB) && on_gpu(matC), "arrays must live on the GPU");
  TF_REQUIRE(matA->ndim == 2 && matB->ndim == 2 && matC->ndim == 2, "operands must be 2-D");
  const int64_t M = matA->shape[transposeA ? 1 : 0], K = matA->shape[transposeA ? 0 : 1];
  const int64_t Kb = matB->shape[transposeB ? 1 : 0], N = matB->shape[transposeB ? 0 : 1];
  TF_REQUIRE(K == Kb, "inner dimensions differ (%lld vs %lld)", (long long)K, (long long)Kb);
  TF_REQUIRE(matC->shape[0] == M && matC->shape[1] == N, "output must be %lld x %lld", (long long)M,
             (long long)N);
  const int64_t a_bytes = numel(matA) * 4, b_bytes = numel(matB) * 4;
  TF_REQUIRE(a_bytes < (1ll << 31) && b_bytes < (1ll << 31) && M * N * 4 < (1ll << 31),
             "operands and results of 2 GiB or more are not supported");
  // the epilogue forms 32-bit byte offsets for every row of a tile, including the rows
  // of the last tile that lie past M (the buffer bound drops them only if the offset
  // has not wrapped)
  TF_REQUIRE((M + 128) * N * 4 < (1ll << 32), "result too wide: (rows + 128) * columns * 4 must stay below 4 GiB");
  hipStream_t s = stream_of(stream);
  if (M == 0 || N == 0) return 0;
  if (K == 0) return DLGpuArraySet(matC, 0.f, stream);

  const int lda = (int)matA->shape[1], ldb = (int)matB->shape[1];
  const bool big = M > 64 && N > 64 && cdiv(M, 128) * cdiv(N, 128) >= num_cus();
  const int bm = big ? 128 : 64, bn = big ? 128 : 64;
  const int tiles = cdiv(M, bm) * cdiv(N, bn);
  const int splits = choose_splits(tiles, (int)K, 256);
  Geometry g = make_geometry((int)M, (int)N, (int)K, bm, bn, splits);
  plan_fold(g, (int)K, big ? 16 : 32, 1);
  FoldBuffers fb;
  if (acquire_fold(g, bm, bn, 1, s, fb) != 0) {  // no scratch (this entry point cannot report it): no fold
    release_fold(fb);
    g = make_geometry((int)M, (int)N, (int)K, bm, bn, splits);
  }

  float *dst = (float *)matC->data;
  float *partial = nullptr;
  if (g.splits > 1) {
    partial = (float *)device_alloc((size_t)g.splits * M * N * sizeof(float));
    if (!partial) {  // no scratch: fall back to one pass over the whole reduction
      g = make_geometry((int)M, (int)N, (int)K, bm, bn, 1);
    } else {
      dst = partial;
    }
  }
  StoreRowMajor ep{dst, (int)N, (int)M, (int)N, M * N};
  if (big)
    dispatch<128, 128, 16>((const float *)matA->data, transposeA, lda, (uint32_t)a_bytes, (const float *)matB->data,
                       transposeB, ldb, (uint32_t)b_bytes, ep, (int)M, (int)N, (int)K, g, s);
  else
    dispatch<64, 64, 32>((const float *)matA->data, transposeA, lda, (uint32_t)a_bytes, (const float *)matB->data,
                     transposeB, ldb, (uint32_t)b_bytes, ep, (int)M, (int)N, (int)K, g, s);
  if (partial) {
    launch_split_sum(partial, (float *)matC->data, M * N, g.splits, s);
    device_free(partial);
  }
  release_fold(fb);
  return finish(s, "DLGpuMatrixMultiply");
}
