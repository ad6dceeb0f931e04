// Device helpers shared by the MFMA kernels for 16-bit inputs (fbla_mfma.hip) and for fp32
// inputs (fbla_mfma32.hip).
#ifndef FBLA_MFMA_SHARED_H
#define FBLA_MFMA_SHARED_H

#include "fbla_kernels.h"

namespace fbla {
namespace mfma {

typedef float f32x16 __attribute__((ext_vector_type(16)));

// Streaming accesses.  Every token row is read once per kernel and every output row written
// once, so the rows bypass the caches' retention ("nt" on the instruction): a kernel that
// starts behind the dirty lines of its predecessor's output then does not wait for their
// write-back on every fill.
template <bool NT, typename V>
__device__ __forceinline__ V stream_load(const void* src) {
  if constexpr (NT) {
    return __builtin_nontemporal_load(reinterpret_cast<const V*>(src));
  } else {
    return *reinterpret_cast<const V*>(src);
  }
}
template <bool NT, typename V>
__device__ __forceinline__ void stream_store(void* dst, V w) {
  if constexpr (NT) {
    __builtin_nontemporal_store(w, reinterpret_cast<V*>(dst));
  } else {
    *reinterpret_cast<V*>(dst) = w;
  }
}

// Orders this wave's LDS traffic: everything written before is visible to every
// lane of the wave after (LDS executes a wave's instructions in order; this keeps
// the compiler from moving accesses across the point).
__device__ __forceinline__ void wave_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// Workgroups are dispatched round-robin over the eight XCDs (workgroup i runs on XCD i % 8).
// In a packed batch the heads of one token sit next to each other in memory, so the workgroups
// of one sequence (its heads and chunks: `per_seq` of them) should run at the same time and
// behind the same L2: workgroup i takes item j of XCD x = i % 8, j = i / 8, and the XCDs take
// the sequences (in walking order) round-robin.  Sequences beyond the last multiple of eight
// keep the plain order.  Returns the item index (sequence rank * per_seq + item within it).
__device__ __forceinline__ int packed_item(const Prob& p, int wg, int per_seq) {
  if (!(p.flags & kXcdOrder)) return wg;
  const int full = (p.N / 8) * 8 * per_seq;
  if (wg >= full) return wg;
  const int xcd = wg & 7, j = wg >> 3;
  return ((j / per_seq) * 8 + xcd) * per_seq + j % per_seq;
}

// Packed sequences have different lengths, and workgroups are dispatched in index
// order: handing out the longest sequences first (LPT) keeps the last round of
// workgroups short.  Returns the index of the sequence with the `rank`-th largest
// length (ties by index): from the order a kernel wrote before (p.perm), else ranked here
// in LDS (quadratic in the number of sequences: small batches only); the identity for dense
// problems, a single sequence, or when neither applies.  Called by all threads of the workgroup.
constexpr int kLptMax = kRankInline;
__device__ __forceinline__ int lpt_sequence(const Prob& p, int rank, int* lens /* [kLptMax + 1] */) {
  if (!p.cu || p.N < 2) return rank;
  if (p.perm) return __builtin_amdgcn_readfirstlane(p.perm[rank]);
  if (p.N > kLptMax) return rank;
  const int nthreads = blockDim.x;
  for (int i = threadIdx.x; i < p.N; i += nthreads) lens[i] = p.cu[i + 1] - p.cu[i];
  __syncthreads();
  for (int j = threadIdx.x; j < p.N; j += nthreads) {
    const int lj = lens[j];
    int r = 0;
    for (int i = 0; i < p.N; ++i) r += (lens[i] > lj) || (lens[i] == lj && i < j);
    if (r == rank) lens[kLptMax] = j;
  }
  __syncthreads();
  return __builtin_amdgcn_readfirstlane(lens[kLptMax]);  // the same for all lanes: keep it scalar
}

// The state kernel's form of the same reduction.  The DK x DV state is tiled into 64 x 64
// blocks; a block is owned by G = 4 / (number of blocks) waves that take interleaved token
// tiles (g = the wave's index inside its group).  The group's accumulators are summed in a
// fixed order through the group's LDS buffer `red` (64 * 66 floats; unused for G = 1) and
// wave g = 0 stores the block: dst points at the block's first element inside the [DK][DV]
// matrix (leading dimension ld), dst_vec (optional) at the block's 64 entries of the vector.
// Register r of accumulator (a,b) is row 2*m + a, column 2*pp + b with
// m = 8*(r/4) + 4*kb + r%4 (PAIRED: lanes own feature pairs, the 16-bit kernels) or row
// 32*a + m, column 32*b + pp (lanes own single features, the fp32 kernels).  Only the first
// `rows_ok` rows and `cols_ok` columns of the block are stored (a head dim that is not a
// multiple of 64 leaves the rest of its last block as padding).  Must be reached by all waves
// of the workgroup.  FOLD = true (PAIRED only): the block holds two 32 x 32 sums on its diagonal
// (rows and columns 0..31 and 32..63) whose sum is stored as a 32 x 32 matrix (rows_ok =
// cols_ok = 32), and likewise the two halves of the vector.
template <int G, bool PAIRED = true, bool FOLD = false>
__device__ __forceinline__ void reduce_store_block(f32x16 (&acc)[2][2], float (&ks)[2], float* red,
                                                   float* dst, int ld, float* dst_vec, float mscale,
                                                   float vscale, int g, int lane, int rows_ok = 64,
                                                   int cols_ok = 64) {
  const int pp = lane & 31, kb = lane >> 5;
  auto spill = [&]() {
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
      for (int b = 0; b < 2; ++b)
#pragma unroll
        for (int r = 0; r < 16; ++r) red[((a * 2 + b) * 16 + r) * 64 + lane] = acc[a][b][r];
#pragma unroll
    for (int a = 0; a < 2; ++a) red[(64 + a) * 64 + lane] = ks[a];
  };
  auto absorb = [&]() {
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
      for (int b = 0; b < 2; ++b)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[a][b][r] += red[((a * 2 + b) * 16 + r) * 64 + lane];
#pragma unroll
    for (int a = 0; a < 2; ++a) ks[a] += red[(64 + a) * 64 + lane];
  };
  if constexpr (G == 4) {  // 2 -> 0, 3 -> 1, 1 -> 0
    if (g == 2) spill();
    __syncthreads();
    if (g == 0) absorb();
    __syncthreads();
    if (g == 3) spill();
    __syncthreads();
    if (g == 1) absorb();
    __syncthreads();
    if (g == 1) spill();
    __syncthreads();
    if (g == 0) absorb();
  } else if constexpr (G == 2) {
    if (g == 1) spill();
    __syncthreads();
    if (g == 0) absorb();
  }
  if (g != 0) return;
  if constexpr (FOLD) {
    // row + 32 is register r + 8, column + 32 is lane + 16
#pragma unroll
    for (int a = 0; a < 2; ++a) {
#pragma unroll
      for (int b = 0; b < 2; ++b)
#pragma unroll
        for (int r = 0; r < 8; ++r) acc[a][b][r] += __shfl_down(acc[a][b][r + 8], 16);
      ks[a] += __shfl_down(ks[a], 16);
    }
  }
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = 8 * (r >> 2) + 4 * kb + (r & 3);
        const int row = PAIRED ? 2 * m + a : 32 * a + m, col = PAIRED ? 2 * pp + b : 32 * b + pp;
        if (row < rows_ok && col < cols_ok) dst[row * ld + col] = acc[a][b][r] * mscale;
      }
  if (dst_vec) {
#pragma unroll
    for (int a = 0; a < 2; ++a) {
      const float tot = ks[a] + __shfl_xor(ks[a], 32);
      const int row = PAIRED ? 2 * pp + a : 32 * a + pp;
      if (kb == 0 && row < rows_ok) dst_vec[row] = tot * vscale;
    }
  }
}

// Byte offset of 16-byte chunk `chunk` of row `row` inside a swizzled tile.  The LDS serves
// 16 lanes x 16 bytes per cycle out of 64 banks, so the reads of one chunk column over 16
// consecutive rows must fall into 16 different 16-byte bank groups: 256-byte rows use all
// four low row bits; 128-byte rows come in pairs that already sit in different halves of
// the banks, so the pair index is used.
template <int ROWB> __device__ __forceinline__ int swz(int row, int chunk) {
  if constexpr (ROWB == 256) return row * ROWB + ((chunk ^ (row & 15)) << 4);
  else if constexpr (ROWB == 128) return row * ROWB + ((chunk ^ ((row >> 1) & 7)) << 4);
  else return row * ROWB + ((chunk ^ (row & 7)) << 4);
}

}  // namespace mfma
}  // namespace fbla
#endif
