// fp32 MFMA tile engine shared by the matrix multiply and the three implicit-GEMM
// convolutions (forward, grad-data, grad-filter).
//
//   D[m, n] = sum_k A(m, k) * B(k, n)
//
// One 256-lane workgroup (four wave64 waves in a 2 x 2 arrangement) owns a
// BM x BN tile of D and walks the reduction in steps of BK (16 or 32, a template
// parameter chosen with the tile shape).  Operand tiles
// are fetched with bounds-checked buffer loads (an out-of-range or padded
// element is given an offset beyond the buffer and reads as zero, so tails and
// convolution padding need no branches), staged through double-buffered LDS as
// [k][m] / [k][n] planes, and consumed by v_mfma_f32_32x32x2_f32: per MFMA a
// lane supplies A[m = lane%32][k = lane/32] and B[k = lane/32][n = lane%32],
// and owns 16 accumulators D[8*(v/4) + 4*(lane/32) + v%4][lane%32].
//
// What differs between the four users is only how a tile element's address is
// formed (the loader) and where an accumulator is written (the epilogue); both
// are template policies defined next to their users.
#pragma once

#include <hip/hip_runtime.h>
#include <cstdint>
#include <type_traits>

namespace tf {
namespace gemm {

typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int THREADS = 256;    // four waves
constexpr int LDS_PAD = 4;      // row padding of the LDS planes (floats)
constexpr uint32_t OOB = 0x80000000u;  // byte offset that every buffer bound check rejects

// Raw buffer resource over [base, base + bytes): loads past `bytes` return 0.
__device__ inline __amdgpu_buffer_rsrc_t make_rsrc(const void *base, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, (int)bytes, 0x00020000);
}
__device__ inline float buf_load(__amdgpu_buffer_rsrc_t r, uint32_t byte_off) {
  return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, (int)byte_off, 0, 0));
}

// Unsigned division by a runtime constant: q = (umulhi(n, mul) + n) >> shift,
// exact for n < 2^31.
struct FastDiv {
  uint32_t d, mul, shift;
  FastDiv() : d(1), mul(0), shift(0) {}
  explicit FastDiv(uint32_t div) : d(div ? div : 1) {
    div = d;
    uint32_t l = 0;
    while ((1ull << l) < div) ++l;
    shift = l;
    mul = (uint32_t)((((1ull << l) - div) << 32) / div + 1);
  }
  __device__ inline uint32_t div(uint32_t n) const { return (__umulhi(n, mul) + n) >> shift; }
  __device__ inline void divmod(uint32_t n, uint32_t &q, uint32_t &r) const {
    q = div(n);
    r = n - q * d;
  }
};

// ---- thread -> tile-element maps ---------------------------------------------
// "Along" map: the 256 lanes run along the tile's m (or n) extent D, so that one
// load instruction of a wave reads 64 consecutive m for a single, wave-uniform k.
template <int D, int BK>
struct AlongMap {
  static_assert(D == 64 || D == 128 || D == 256, "tile extent");
  static constexpr int KSTEP = THREADS / D;  // k rows covered per pass
  static constexpr int EPT = BK / KSTEP;     // elements per thread per stage
  int d_local;                               // position along the tile extent
  int k_first;                               // wave-uniform
  __device__ inline void init(int tid) {
    d_local = tid % D;
    k_first = __builtin_amdgcn_readfirstlane(tid / D);
  }
  __device__ inline int k_of(int e) const { return k_first + e * KSTEP; }
};

// "Across" map: BK consecutive lanes run along k (the contiguous direction of
// the operand in memory), the remaining lane groups along the tile extent.
template <int D, int BK>
struct AcrossMap {
  static_assert(D % (THREADS / BK) == 0, "tile extent");
  static constexpr int DSTEP = THREADS / BK;
  static constexpr int EPT = D / DSTEP;
  int k_local;
  int d_first;
  __device__ inline void init(int tid) {
    k_local = tid % BK;
    d_first = tid / BK;
  }
  __device__ inline int d_of(int e) const { return d_first + e * DSTEP; }
};

// ---- plain row-major matrix operands -------------------------------------------
// element(d, k) = base[k * ld + d]        (tile extent contiguous in memory)
template <int D, int BK>
struct PlainAlong {
  using Map = AlongMap<D, BK>;
  static constexpr int EPT = Map::EPT;
  const float *base;
  uint32_t bytes;
  int ld, d_extent, k_extent;

  struct State {
    Map map;
    __amdgpu_buffer_rsrc_t rsrc;
    uint32_t d_off;  // byte offset of this lane's d, or OOB
  };
  __device__ inline void init(State &st, int origin, int tid) const {
    st.map.init(tid);
    st.rsrc = make_rsrc(base, bytes);
    const int d = origin + st.map.d_local;
    st.d_off = d < d_extent ? (uint32_t)d * 4u : OOB;
  }
  // k_limit: first reduction index this workgroup must not read (<= k_extent)
  __device__ inline void load(const State &st, int k0, int k_limit, float (&reg)[EPT]) const {
#pragma unroll
    for (int e = 0; e < EPT; ++e) {
      const int k = k0 + st.map.k_of(e);
      const uint32_t off = k < k_limit ? st.d_off + (uint32_t)k * (uint32_t)ld * 4u : OOB;
      reg[e] = buf_load(st.rsrc, off | (st.d_off & OOB));
    }
  }
  template <int LD>
  __device__ inline void store(const State &st, float (*tile)[LD], const float (&reg)[EPT]) const {
#pragma unroll
    for (int e = 0; e < EPT; ++e) tile[st.map.k_of(e)][st.map.d_local] = reg[e];
  }
};

// element(d, k) = base[d * ld + k]        (reduction contiguous in memory)
template <int D, int BK>
struct PlainAcross {
  using Map = AcrossMap<D, BK>;
  static constexpr int EPT = Map::EPT;
  const float *base;
  uint32_t bytes;
  int ld, d_extent, k_extent;

  struct State {
    Map map;
    __amdgpu_buffer_rsrc_t rsrc;
    uint32_t row_off[EPT];  // byte offset of row d, or OOB
  };
  __device__ inline void init(State &st, int origin, int tid) const {
    st.map.init(tid);
    st.rsrc = make_rsrc(base, bytes);
#pragma unroll
    for (int e = 0; e < EPT; ++e) {
      const int d = origin + st.map.d_of(e);
      st.row_off[e] = d < d_extent ? (uint32_t)d * (uint32_t)ld * 4u : OOB;
    }
  }
  __device__ inline void load(const State &st, int k0, int k_limit, float (&reg)[EPT]) const {
    const int k = k0 + st.map.k_local;
    const uint32_t k_off = k < k_limit ? (uint32_t)k * 4u : OOB;
#pragma unroll
    for (int e = 0; e < EPT; ++e) reg[e] = buf_load(st.rsrc, (st.row_off[e] + k_off) | ((st.row_off[e] | k_off) & OOB));
  }
  template <int LD>
  __device__ inline void store(const State &st, float (*tile)[LD], const float (&reg)[EPT]) const {
#pragma unroll
    for (int e = 0; e < EPT; ++e) tile[st.map.k_local][st.map.d_of(e)] = reg[e];
  }
};

// ---- 16-byte loaders ---------------------------------------------------------------
// One buffer_load_dwordx4 per lane fetches four consecutive elements: a quarter of
// the load instructions and of the address arithmetic of the one-element loaders
// above.  Addressing is segmented so that the same two loaders serve plain
// matrices and the NCHW tensors of 1x1 / stride-1 convolutions (pixels of one image
// and channel are contiguous, images are `outer` elements apart):
//   Along4 :  element(d, k) = base[(d / inner) * outer + d % inner + k * ld]
//   Across4:  element(d, k) = base[d * ld + (k / inner) * outer + k % inner]
// A plain matrix is the case inner = 2^31 (one segment), outer = 0.
// Preconditions, checked by the callers: base 16-byte aligned; ld, inner and outer
// multiples of 4; the extent along the vectorised direction (d for Along4, k for
// Across4) a multiple of 4, so that a vector is entirely inside or outside.
//
// Ragged segments: a segment whose real length is not a multiple of 4 (the 49 pixels
// of a 7x7 map) is addressed with `inner` rounded up to the next multiple of 4 while
// `outer` stays the real distance between segments.  The last vector of a segment
// then also fetches up to three elements that belong to what follows it in memory
// (4-byte aligned 16-byte loads are fine for global memory).  For Along4 they land in
// tile columns that exist only in the padded index space and are dropped by the
// epilogue; for Across4 they would enter the reduction, so its RAGGED form zeroes
// every element whose position in the segment is `seg_valid` or more.
typedef float f32x4v __attribute__((ext_vector_type(4)));
constexpr uint32_t ONE_SEGMENT = 0x80000000u;
__device__ inline f32x4v buf_load4(__amdgpu_buffer_rsrc_t r, uint32_t byte_off) {
  return __builtin_bit_cast(f32x4v, __builtin_amdgcn_raw_buffer_load_b128(r, (int)byte_off, 0, 0));
}
inline bool vec4_ok(const void *base, int64_t a, int64_t b = 0, int64_t c = 0, int64_t d = 0) {
  return (reinterpret_cast<uintptr_t>(base) & 15u) == 0 && a % 4 == 0 && b % 4 == 0 && c % 4 == 0 && d % 4 == 0;
}

template <int D, int BK>
struct Along4 {
  static constexpr int LPR = D / 4;             // lanes per k row of the tile
  static constexpr int KSTEP = THREADS / LPR;   // k rows covered per pass
  static constexpr int VPT = BK / KSTEP;        // vector loads per lane per stage
  static constexpr int EPT = VPT * 4;
  static_assert(VPT >= 1 && VPT * KSTEP == BK, "tile shape");
  const float *base;
  uint32_t bytes;
  int ld, d_extent, k_extent;
  FastDiv div_inner;
  int outer;

  struct State {
    __amdgpu_buffer_rsrc_t rsrc;
    uint32_t d_off;  // byte offset of this lane's first d, or OOB
    int d_local, k_first;
  };
  __device__ inline void init(State &st, int origin, int tid) const {
    st.rsrc = make_rsrc(base, bytes);
    st.d_local = (tid % LPR) * 4;
    st.k_first = tid / LPR;
    const int d = origin + st.d_local;
    uint32_t seg, rem;
    div_inner.divmod((uint32_t)(d < d_extent ? d : 0), seg, rem);
    st.d_off = d < d_extent ? (seg * (uint32_t)outer + rem) * 4u : OOB;
  }
  __device__ inline void load(const State &st, int k0, int k_limit, float (&reg)[EPT]) const {
#pragma unroll
    for (int e = 0; e < VPT; ++e) {
      const int k = k0 + st.k_first + e * KSTEP;
      const uint32_t off = k < k_limit ? st.d_off + (uint32_t)k * (uint32_t)ld * 4u : OOB;
      const f32x4v v = buf_load4(st.rsrc, off | (st.d_off & OOB));
#pragma unroll
      for (int i = 0; i < 4; ++i) reg[4 * e + i] = v[i];
    }
  }
  template <int LD>
  __device__ inline void store(const State &st, float (*tile)[LD], const float (&reg)[EPT]) const {
    static_assert(LD % 4 == 0, "rows of the LDS plane must keep 16-byte alignment");
#pragma unroll
    for (int e = 0; e < VPT; ++e) {
      const f32x4v v = {reg[4 * e], reg[4 * e + 1], reg[4 * e + 2], reg[4 * e + 3]};
      *reinterpret_cast<f32x4v *>(&tile[st.k_first + e * KSTEP][st.d_local]) = v;
    }
  }
};

template <int D, int BK, bool RAGGED = false>
struct Across4 {
  static constexpr int LPR = BK / 4;            // lanes per d row of the tile
  static constexpr int DSTEP = THREADS / LPR;
  static constexpr int VPT = D / DSTEP;
  static constexpr int EPT = VPT * 4;
  static_assert(VPT >= 1 && VPT * DSTEP == D, "tile shape");
  // The four consecutive reduction elements a lane fetches stay together in LDS: the
  // plane is [d][k] (see gemm_kernel), written with one 16-byte store per vector.
  static constexpr bool kKContig = true;
  const float *base;
  uint32_t bytes;
  int ld, d_extent, k_extent;
  FastDiv div_inner;
  int outer;
  int seg_valid = 0;  // RAGGED: real length of a segment

  struct State {
    __amdgpu_buffer_rsrc_t rsrc;
    uint32_t row_off[VPT];  // byte offset of row d, or OOB
    int k_local, d_first;
  };
  __device__ inline void init(State &st, int origin, int tid) const {
    st.rsrc = make_rsrc(base, bytes);
    st.k_local = (tid % LPR) * 4;
    st.d_first = tid / LPR;
#pragma unroll
    for (int e = 0; e < VPT; ++e) {
      const int d = origin + st.d_first + e * DSTEP;
      st.row_off[e] = d < d_extent ? (uint32_t)d * (uint32_t)ld * 4u : OOB;
    }
  }
  __device__ inline void load(const State &st, int k0, int k_limit, float (&reg)[EPT]) const {
    const int k = k0 + st.k_local;
    uint32_t seg, rem;
    div_inner.divmod((uint32_t)(k < k_limit ? k : 0), seg, rem);
    const uint32_t k_off = k < k_limit ? (seg * (uint32_t)outer + rem) * 4u : OOB;
#pragma unroll
    for (int e = 0; e < VPT; ++e) {
      const f32x4v v = buf_load4(st.rsrc, (st.row_off[e] + k_off) | ((st.row_off[e] | k_off) & OOB));
#pragma unroll
      for (int i = 0; i < 4; ++i) reg[4 * e + i] = (RAGGED && (int)rem + i >= seg_valid) ? 0.f : v[i];
    }
  }
  template <int LD>
  __device__ inline void store(const State &st, float (*tile)[LD], const float (&reg)[EPT]) const {
    static_assert(LD % 4 == 0, "rows of the LDS plane must keep 16-byte alignment");
#pragma unroll
    for (int e = 0; e < VPT; ++e) {
      const f32x4v v = {reg[4 * e], reg[4 * e + 1], reg[4 * e + 2], reg[4 * e + 3]};
      *reinterpret_cast<f32x4v *>(&tile[st.d_first + e * DSTEP][st.k_local]) = v;
    }
  }
};

template <class L, class = void>
struct lds_k_contig : std::false_type {};
template <class L>
struct lds_k_contig<L, std::enable_if_t<L::kKContig>> : std::true_type {};

// ---- epilogue: plain row-major store ---------------------------------------------
// Stores go through a buffer descriptor over this split's output: a row past
// m_extent lies outside the buffer by itself, a column past n_extent is given an
// out-of-range offset, and the hardware drops both -- no branch around the
// store and 32-bit offset arithmetic only.
__device__ inline void buf_store(__amdgpu_buffer_rsrc_t r, uint32_t byte_off, float v) {
  __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(int, v), r, (int)byte_off, 0, 0);
}
struct StoreRowMajor {
  float *out;
  int ld, m_extent, n_extent;
  int64_t split_stride;  // elements between the outputs of consecutive k-splits
  struct State {
    __amdgpu_buffer_rsrc_t rsrc;
  };
  template <int TN>
  __device__ inline void init(State &st, int /*n0*/, int /*lane*/, int split) const {
    st.rsrc = make_rsrc(out + (int64_t)split * split_stride, (uint32_t)m_extent * (uint32_t)ld * 4u);
  }
  __device__ inline void store(const State &st, int m, int n, int /*j*/, float v) const {
    const uint32_t off = ((uint32_t)m * (uint32_t)ld + (uint32_t)n) * 4u;
    buf_store(st.rsrc, n < n_extent ? off : OOB, v);
  }
};

// ---- in-kernel fold of k-split tiles ---------------------------------------------------
// Some output tiles of a launch can be computed by several workgroups ("pieces"),
// each over its own range of the reduction, without a second pass: a piece
// writes its raw accumulators to scratch, takes a ticket for its tile, and the
// piece that draws the last ticket adds all pieces of the tile in piece order
// (its own included, re-read from scratch) and runs the epilogue.  The order of
// the additions is fixed, so the result does not depend on which piece arrives
// last.  Nobody waits for anybody: a piece that is not last simply exits.
// Used in two ways by the hosts:
//   * every tile folded (first_tile = 0): a k-split of a few pieces without the
//     separate sum pass;
//   * only the tiles past the last full round over the CUs folded: the remainder
//     round, which would keep a fraction of the CUs busy for a whole tile time,
//     becomes about one short piece per CU.
struct Fold {
  float *scratch;      // [batch][folded tile][piece][BM * BN] accumulators, lane-major
  unsigned *tickets;   // [batch][folded tile], zero before the launch; the last piece zeroes its counter again
  int first_tile;      // tiles [0, first_tile) are plain, tiles [first_tile, tiles) are folded
  int plain_blocks;    // workgroups of the plain tiles (first_tile * plain splits); they come first in the grid
  int pieces;          // workgroups per folded tile; 0 or 1: nothing is folded
  int k_per_piece;     // reduction steps per piece (a multiple of BK)
};

// Hardware hands consecutive workgroup ids to the 8 XCDs round-robin; this gives
// each XCD a contiguous range of the n logical ids instead.
__device__ inline int xcd_contiguous(int id, int n) {
  const int per_xcd = n >> 3;
  return id < (per_xcd << 3) ? (id & 7) * per_xcd + (id >> 3) : id;
}

// ---- the kernel ----------------------------------------------------------------------
// Work decomposition: gridDim.x = tiles_m * tiles_n * splits (plus, with a fold, the
// pieces of the folded tiles behind the plain workgroups).  Hardware hands
// consecutive workgroup ids to the 8 XCDs round-robin; the remap below gives
// each XCD a contiguous range of logical tile ids, ordered m-fastest, so the
// workgroups that share one B tile (the large, gathered operand) also share an
// L2.  Every wave executes the same number of barriers and exits after its
// epilogue; there is no data-dependent loop.
template <int BM, int BN, int BK, class ALoader, class BLoader, class Epilogue>
__global__ __launch_bounds__(THREADS) void gemm_kernel(const ALoader al, const BLoader bl, const Epilogue ep,
                                                      int k_extent, int k_per_split, int tiles_m, int tiles_n,
                                                      const Fold fold) {
  constexpr int WM = BM / 2, WN = BN / 2;  // wave tile
  constexpr int TM = WM / 32, TN = WN / 32;
  static_assert(TM >= 1 && TN >= 1, "tile too small for a 2x2 wave grid");
  // LDS planes.  An operand whose loader fetches along the reduction (kKContig) is kept
  // as [m][k]: its vectors go to LDS untransposed, and a lane fetches the four
  // reduction elements of four consecutive MFMAs with one 16-byte read.  For that the
  // reduction is walked in a permuted order inside every group of eight: MFMA s of the
  // group takes k = 8g + s from lanes 0..31 and k = 8g + 4 + s from lanes 32..63, for
  // both operands alike (a sum does not care).  Without such an operand the planes are
  // [k][m] / [k][n] and the order is the plain one.
  constexpr bool AKC = lds_k_contig<ALoader>::value, BKC = lds_k_contig<BLoader>::value;
  constexpr bool PERM = AKC || BKC;
  static_assert(!PERM || BK % 8 == 0, "groups of eight reduction elements");
  constexpr int LDK = BK + LDS_PAD;
  constexpr int LDA = AKC ? LDK : BM + LDS_PAD, ROWS_A = AKC ? BM : BK;
  constexpr int LDB = BKC ? LDK : BN + LDS_PAD, ROWS_B = BKC ? BN : BK;
  __shared__ float As[2][ROWS_A][LDA];
  __shared__ float Bs[2][ROWS_B][LDB];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave & 1, wn = wave >> 1;

  // which tile, and which part of the reduction (all of this is scalar arithmetic)
  const int tiles = tiles_m * tiles_n;
  const bool folding = fold.pieces > 1;
  const bool folded = folding && (int)blockIdx.x >= fold.plain_blocks;
  int tile, split, k_begin, k_end, fold_tile = 0, piece = 0;
  if (!folded) {
    const int plain_tiles = folding ? fold.first_tile : tiles;
    const int logical = xcd_contiguous((int)blockIdx.x, folding ? fold.plain_blocks : (int)gridDim.x);
    tile = logical % plain_tiles;
    split = logical / plain_tiles;
    k_begin = split * k_per_split;
    k_end = k_begin + k_per_split;
  } else {
    const int fold_tiles = tiles - fold.first_tile;
    const int logical = xcd_contiguous((int)blockIdx.x - fold.plain_blocks, (int)gridDim.x - fold.plain_blocks);
    fold_tile = logical % fold_tiles;
    piece = logical / fold_tiles;
    tile = fold.first_tile + fold_tile;
    split = 0;
    k_begin = piece * fold.k_per_piece;
    k_end = k_begin + fold.k_per_piece;
  }
  if (k_end > k_extent) k_end = k_extent;
  const int tm = tile % tiles_m, tn = tile / tiles_m;
  const int m0 = tm * BM, n0 = tn * BN;

  typename ALoader::State sa;
  typename BLoader::State sb;
  al.init(sa, m0, tid);
  bl.init(sb, n0, tid);

  f32x16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  float ra[ALoader::EPT], rb[BLoader::EPT];
  al.load(sa, k_begin, k_end, ra);
  bl.load(sb, k_begin, k_end, rb);
  al.template store<LDA>(sa, As[0], ra);
  bl.template store<LDB>(sb, Bs[0], rb);
  __syncthreads();

  const int lrow = lane >> 5;   // which of the two k of an MFMA this lane feeds
  const int lcol = lane & 31;
  int buf = 0;
  for (int k0 = k_begin; k0 < k_end; k0 += BK) {
    // Fetch the next stage while this one is multiplied.  Past the end of the
    // range every offset is out of bounds, so the last iteration's fetch costs no
    // memory traffic and the loop body has no branch: loads, address arithmetic
    // and MFMAs of one iteration are free to interleave.
    al.load(sa, k0 + BK, k_end, ra);
    bl.load(sb, k0 + BK, k_end, rb);
    // keep the fetches ahead of the multiply: without this fence the scheduler
    // sinks them next to their use and their latency is no longer hidden
    __builtin_amdgcn_sched_barrier(0);
    // MFMA operands are read from LDS one sub-step ahead of the MFMAs that use
    // them (two register sets), so the LDS latency sits under the previous
    // sub-step's matrix instructions.
    if constexpr (PERM) {
      // fragments of a whole group (four MFMA steps) per fetch, one group ahead
      f32x4v a4[2][TM], b4[2][TN];
      auto fetch_group = [&](int gi, int slot) {
#pragma unroll
        for (int i = 0; i < TM; ++i) {
          const int m = wm * WM + 32 * i + lcol;
          if constexpr (AKC) {
            a4[slot][i] = *reinterpret_cast<const f32x4v *>(&As[buf][m][8 * gi + 4 * lrow]);
          } else {
#pragma unroll
            for (int s = 0; s < 4; ++s) a4[slot][i][s] = As[buf][8 * gi + 4 * lrow + s][m];
          }
        }
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          const int n = wn * WN + 32 * j + lcol;
          if constexpr (BKC) {
            b4[slot][j] = *reinterpret_cast<const f32x4v *>(&Bs[buf][n][8 * gi + 4 * lrow]);
          } else {
#pragma unroll
            for (int s = 0; s < 4; ++s) b4[slot][j][s] = Bs[buf][8 * gi + 4 * lrow + s][n];
          }
        }
      };
      fetch_group(0, 0);
#pragma unroll
      for (int gi = 0; gi < BK / 8; ++gi) {
        const int cur = gi & 1, nxt = cur ^ 1;
        if (gi + 1 < BK / 8) fetch_group(gi + 1, nxt);
#pragma unroll
        for (int s = 0; s < 4; ++s)
#pragma unroll
          for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
              acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a4[cur][i][s], b4[cur][j][s], acc[i][j], 0, 0, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
      al.template store<LDA>(sa, As[buf ^ 1], ra);
      bl.template store<LDB>(sb, Bs[buf ^ 1], rb);
      __syncthreads();
      buf ^= 1;
      continue;
    }
    float a[2][TM], b[2][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i) a[0][i] = As[buf][lrow][wm * WM + 32 * i + lcol];
#pragma unroll
    for (int j = 0; j < TN; ++j) b[0][j] = Bs[buf][lrow][wn * WN + 32 * j + lcol];
#pragma unroll
    for (int kk = 0; kk < BK / 2; ++kk) {
      const int cur = kk & 1, nxt = cur ^ 1;
      if (kk + 1 < BK / 2) {
        const int krow = 2 * (kk + 1) + lrow;
#pragma unroll
        for (int i = 0; i < TM; ++i) a[nxt][i] = As[buf][krow][wm * WM + 32 * i + lcol];
#pragma unroll
        for (int j = 0; j < TN; ++j) b[nxt][j] = Bs[buf][krow][wn * WN + 32 * j + lcol];
      }
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[cur][i], b[cur][j], acc[i][j], 0, 0, 0);
    }
#pragma unroll
    for (int kk = 0; kk < BK / 2 - 1; ++kk) {
      __builtin_amdgcn_sched_group_barrier(0x100, TM + TN, 0);  // LDS reads of sub-step kk+1
      __builtin_amdgcn_sched_group_barrier(0x008, TM * TN, 0);  // MFMAs of sub-step kk
    }
    __builtin_amdgcn_sched_barrier(0);
    al.template store<LDA>(sa, As[buf ^ 1], ra);
    bl.template store<LDB>(sb, Bs[buf ^ 1], rb);
    __syncthreads();
    buf ^= 1;
  }

  if (folded) {  // uniform over the workgroup
    // The pieces travel through scratch with device-scope ("sc1") stores and loads:
    // such an access is coherent across the XCDs' L2s by itself, so no cache-wide
    // write-back or invalidate is needed (a __threadfence() here costs exactly that
    // and slows every workgroup of the XCD down).  Ordering: all stores of the piece
    // have been acknowledged (s_waitcnt 0) before the barrier that precedes the ticket.
    constexpr int SC1 = 16;  // device scope in the cache-policy operand of the buffer instructions
    // the flag lives in the first word of the A planes, which nobody reads any more (every
    // wave has passed the barrier that ended the reduction loop): the two 128 x 128 planes
    // of [m][k] operands fill a quarter of a CU's LDS to the byte, and four workgroups
    // per CU are what the kernel is tuned for
    unsigned &is_last = *reinterpret_cast<unsigned *>(&As[0][0][0]);
    const int fold_tiles = tiles - fold.first_tile;
    const size_t slot = (size_t)blockIdx.y * fold_tiles + fold_tile;
    constexpr uint32_t kPieceBytes = (uint32_t)(BM * BN) * 4u;
    const __amdgpu_buffer_rsrc_t pieces_of_tile =
        make_rsrc(fold.scratch + slot * fold.pieces * (size_t)(BM * BN), (uint32_t)fold.pieces * kPieceBytes);
    const uint32_t lane_off = (uint32_t)tid * 16u;
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const f32x4v v = {acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]};
          __builtin_amdgcn_raw_buffer_store_b128(
              __builtin_bit_cast(__attribute__((__vector_size__(4 * sizeof(unsigned)))) unsigned, v), pieces_of_tile,
              (int)((uint32_t)piece * kPieceBytes + (uint32_t)((i * TN + j) * 4 + q) * (THREADS * 16u) + lane_off), 0,
              SC1);
        }
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    if (tid == 0) is_last = atomicAdd(fold.tickets + slot, 1u) == (unsigned)(fold.pieces - 1);
    __syncthreads();
    if (!is_last) return;
    // Last piece of the tile: add the pieces in piece order, four accumulator
    // registers at a time (the sums go straight to the epilogue, so the fold needs
    // no registers beyond the loads in flight), and clear the ticket.
    typename Epilogue::State sf;
    ep.template init<TN>(sf, n0 + wn * WN, lane, 0);
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        f32x4v sum[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) sum[q] = f32x4v{0.f, 0.f, 0.f, 0.f};
        for (int p = 0; p < fold.pieces; ++p) {
          f32x4v part[4];
#pragma unroll
          for (int q = 0; q < 4; ++q)
            part[q] = __builtin_bit_cast(
                f32x4v, __builtin_amdgcn_raw_buffer_load_b128(
                            pieces_of_tile,
                            (int)((uint32_t)p * kPieceBytes + (uint32_t)((i * TN + j) * 4 + q) * (THREADS * 16u) + lane_off),
                            0, SC1));
#pragma unroll
          for (int q = 0; q < 4; ++q) sum[q] += part[q];
        }
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int m = m0 + wm * WM + 32 * i + 8 * (v >> 2) + 4 * lrow + (v & 3);
          const int n = n0 + wn * WN + 32 * j + lcol;
          ep.store(sf, m, n, j, sum[v >> 2][v & 3]);
        }
      }
    if (tid == 0) fold.tickets[slot] = 0u;  // ready for the next launch on this stream
    return;
  }

  typename Epilogue::State se;
  ep.template init<TN>(se, n0 + wn * WN, lane, split);
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int m = m0 + wm * WM + 32 * i + 8 * (v >> 2) + 4 * lrow + (v & 3);
        const int n = n0 + wn * WN + 32 * j + lcol;
        ep.store(se, m, n, j, acc[i][j][v]);
      }
}

// Host-side launch geometry shared by the users.
struct Geometry {
  int tiles_m, tiles_n, splits, k_per_split;
  // in-kernel fold (see Fold): tiles from fold_first_tile on are computed by fold_pieces
  // workgroups each; fold_pieces <= 1: none
  int fold_first_tile = 0, fold_pieces = 0, fold_k_per_piece = 0;
  int tiles() const { return tiles_m * tiles_n; }
  int folded_tiles() const { return fold_pieces > 1 ? tiles() - fold_first_tile : 0; }
  int plain_blocks() const { return (fold_pieces > 1 ? fold_first_tile : tiles()) * splits; }
  unsigned blocks() const { return (unsigned)(plain_blocks() + folded_tiles() * fold_pieces); }
  size_t fold_scratch_bytes(int bm, int bn, int batch = 1) const {
    return (size_t)batch * folded_tiles() * fold_pieces * bm * bn * sizeof(float);
  }
  float *fold_scratch = nullptr;        // set by the host once the buffers are there
  unsigned *fold_ticket_words = nullptr;
  Fold fold() const {
    if (fold_pieces <= 1) return Fold{nullptr, nullptr, 0, 0, 0, 0};
    return Fold{fold_scratch, fold_ticket_words, fold_first_tile, plain_blocks(), fold_pieces, fold_k_per_piece};
  }
};
inline Geometry make_geometry(int M, int N, int K, int bm, int bn, int splits, int BK = 32) {
  Geometry g;
  g.tiles_m = (M + bm - 1) / bm;
  g.tiles_n = (N + bn - 1) / bn;
  if (splits < 1) splits = 1;
  int kps = ((K + splits - 1) / splits + BK - 1) / BK * BK;
  if (kps < BK) kps = BK;
  g.k_per_split = kps;
  g.splits = (K + kps - 1) / kps;
  if (g.splits < 1) g.splits = 1;
  return g;
}

}  // namespace gemm
}  // namespace tf
