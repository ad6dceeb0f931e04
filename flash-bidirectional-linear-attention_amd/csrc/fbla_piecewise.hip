// Piecewise (PISA) attention, forward only: block statistics for the linear
// branch and the attention kernel itself.
//
// chunk statistics (replaces fused_chunk_reduce_kernel,
// flash_bla/ops/piecewise_attn/kernel.py:89-128,152-176):
//   qc_c, kc_c = mean over chunk c of q, k;  vc_c = sum over chunk c of v
//   H = sum_c (K_c - kc_c)^T V_c = K^T V - sum_c kc_c vc_c^T
// K^T V comes from the state kernel (per-chunk partials, fixed-order sum); the
// chunk sums from one streaming kernel; nothing of size [NT, K, V] is
// materialised unless the optional bias (per-chunk norm of (K_c - kc_c)^T V_c)
// is requested.
#include <algorithm>
#include <type_traits>

#include "fbla_kernels.h"

namespace fbla {
namespace piecewise {

constexpr int kThreads = 256;

// One wave per (head, chunk, tensor): lanes own feature pairs, rows are summed in
// fp32 with four rows in flight.  out[(bh*NT + c)*D + d] = sum (or mean).
template <typename T>
__global__ __launch_bounds__(kThreads) void chunk_sums_kernel(
    const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v, float* __restrict__ qc,
    float* __restrict__ kc, float* __restrict__ vc, int64_t BH, int Tn, int NT, int chunk, int K, int V) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int64_t item = (int64_t)blockIdx.x * 4 + wave;  // (bh, c, which)
  if (item >= BH * NT * 3) return;
  const int which = (int)(item % 3);
  const int64_t bc = item / 3;
  const int c = (int)(bc % NT);
  const int64_t bh = bc / NT;
  const int D = which == 2 ? V : K;
  const T* src = (which == 0 ? q : which == 1 ? k : v) + (bh * Tn + (int64_t)c * chunk) * D;
  float* dst = (which == 0 ? qc : which == 1 ? kc : vc) + bc * D;
  const int n = min(chunk, Tn - c * chunk);
  for (int d = lane; d < D; d += 64) {
    float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
    int t = 0;
    for (; t + 4 <= n; t += 4) {
      a0 += to_f32(__builtin_nontemporal_load(src + (int64_t)t * D + d));
      a1 += to_f32(__builtin_nontemporal_load(src + (int64_t)(t + 1) * D + d));
      a2 += to_f32(__builtin_nontemporal_load(src + (int64_t)(t + 2) * D + d));
      a3 += to_f32(__builtin_nontemporal_load(src + (int64_t)(t + 3) * D + d));
    }
    for (; t < n; ++t) a0 += to_f32(src[(int64_t)t * D + d]);
    const float s = (a0 + a1) + (a2 + a3);
    dst[d] = which == 2 ? s : s / (float)n;
  }
}

// The same for 16-bit inputs with D in {64, 128}: 16-byte loads, a lane owns one
// 8-feature column group and every (64 / chunks-per-row)-th row, lanes are combined by
// shuffles at the end.
typedef uint32_t u32x4s __attribute__((ext_vector_type(4)));
template <typename T, int D>
__global__ __launch_bounds__(kThreads) void chunk_sums16_kernel(
    const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v, float* __restrict__ qc,
    float* __restrict__ kc, float* __restrict__ vc, int64_t BH, int Tn, int NT, int chunk, int nten) {
  // nten = 3: q, k and v; nten = 1: q only (k and v statistics come from the state kernel)
  constexpr int CH = D / 8, RPI = 64 / CH;  // chunks per row, rows per wave instruction
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int64_t item = (int64_t)blockIdx.x * 4 + wave;
  if (item >= BH * NT * nten) return;
  const int which = (int)(item % nten);
  const int64_t bc = item / nten;
  const int c = (int)(bc % NT);
  const int64_t bh = bc / NT;
  const T* src = (which == 0 ? q : which == 1 ? k : v) + (bh * Tn + (int64_t)c * chunk) * D;
  float* dst = (which == 0 ? qc : which == 1 ? kc : vc) + bc * D;
  const int n = min(chunk, Tn - c * chunk);
  const int ch = lane % CH, r0 = lane / CH;
  float acc[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) acc[i] = 0.f;
  // 32 rows per trip: half a chunk of the usual size is in flight before the first sum (a whole
  // one costs so many registers that the 6144 waves of a B1-H24-T16384 problem no longer fit the GPU at once)
  constexpr int NLD = 32 / RPI;
  for (int base = 0; base < n; base += 32) {
    u32x4s w[NLD];
#pragma unroll
    for (int u = 0; u < NLD; ++u) {
      const int row = base + u * RPI + r0;
      // (streaming hint: every row is read once here)
      w[u] = row < n ? __builtin_nontemporal_load(reinterpret_cast<const u32x4s*>(src + (int64_t)row * D + ch * 8))
                     : u32x4s{0u, 0u, 0u, 0u};
    }
#pragma unroll
    for (int u = 0; u < NLD; ++u)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        acc[2 * i] += (float)__builtin_bit_cast(T, (uint16_t)(w[u][i] & 0xffffu));
        acc[2 * i + 1] += (float)__builtin_bit_cast(T, (uint16_t)(w[u][i] >> 16));
      }
  }
#pragma unroll
  for (int off = CH; off < 64; off <<= 1)
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] += __shfl_xor(acc[i], off);
  if (lane < CH) {
    const float f = which == 2 ? 1.f : 1.f / (float)n;
#pragma unroll
    for (int i = 0; i < 8; ++i) dst[ch * 8 + i] = acc[i] * f;
  }
}

// H[bh][dk][dv] = sum_p partial_p[dk][dv] - sum_c kc_c[dk] * vc_c[dv]   (kc the MEAN and vc
// the SUM of chunk c, so their product is the whole correction of that chunk).
// One workgroup per (head, 32x32 tile of H); a thread owns a 2x2 patch.  The chunk
// statistics go through LDS in slabs of 128 chunks (coalesced loads, every value is
// then used 16 times from LDS); the chunk order of the sum is fixed.
constexpr int kHTile = 32, kHSlab = 128;
__global__ __launch_bounds__(kThreads) void finish_h_kernel(
    const float* __restrict__ partial, int nparts, const float* __restrict__ kc,
    const float* __restrict__ vc, float* __restrict__ h, int NT, int K, int V) {
  __shared__ float ks[kHSlab][kHTile + 1];
  __shared__ float vs[kHSlab][kHTile + 1];
  const int tk = (K + kHTile - 1) / kHTile, tv = (V + kHTile - 1) / kHTile;
  const int tile = blockIdx.x % (tk * tv);
  const int64_t bh = blockIdx.x / (tk * tv);
  const int dk0 = (tile / tv) * kHTile, dv0 = (tile % tv) * kHTile;
  const int ty = threadIdx.x / 16, tx = threadIdx.x % 16;  // patch rows 2ty.., cols tx, tx+16
  const float* kch = kc + bh * NT * K;
  const float* vch = vc + bh * NT * V;
  float c00 = 0.f, c01 = 0.f, c10 = 0.f, c11 = 0.f;
  for (int cb = 0; cb < NT; cb += kHSlab) {
    const int nc = min(kHSlab, NT - cb);
    __syncthreads();
    // all of a thread's loads are issued before the first is used (clamped addresses instead of
    // branches: a loop of guarded loads waits for every single one)
    constexpr int NF = kHSlab * kHTile / kThreads;
    float kr[NF], vr[NF];
#pragma unroll
    for (int u = 0; u < NF; ++u) {
      const int i = threadIdx.x + u * kThreads, c = i / kHTile, d = i % kHTile;
      const bool kin = c < nc && dk0 + d < K, vin = c < nc && dv0 + d < V;
      kr[u] = kch[kin ? (int64_t)(cb + c) * K + dk0 + d : 0];
      vr[u] = vch[vin ? (int64_t)(cb + c) * V + dv0 + d : 0];
      kr[u] = kin ? kr[u] : 0.f;
      vr[u] = vin ? vr[u] : 0.f;
    }
#pragma unroll
    for (int u = 0; u < NF; ++u) {
      const int i = threadIdx.x + u * kThreads, c = i / kHTile, d = i % kHTile;
      ks[c][d] = kr[u];
      vs[c][d] = vr[u];
    }
    __syncthreads();
#pragma unroll 8
    for (int c = 0; c < kHSlab; ++c) {
      const float k0 = ks[c][2 * ty], k1 = ks[c][2 * ty + 1];
      const float v0 = vs[c][tx], v1 = vs[c][tx + 16];
      c00 = fmaf(k0, v0, c00);
      c01 = fmaf(k0, v1, c01);
      c10 = fmaf(k1, v0, c10);
      c11 = fmaf(k1, v1, c11);
    }
  }
  const int E = K * V, stride = E + K;
  // the four partial sums advance together, four partials per trip: sixteen independent
  // loads in flight instead of one (the order of each sum stays p = 0, 1, 2, ...)
  const int dk_a = dk0 + 2 * ty, dv_a = dv0 + tx;
  const bool ok[2][2] = {{dk_a < K && dv_a < V, dk_a < K && dv_a + 16 < V},
                         {dk_a + 1 < K && dv_a < V, dk_a + 1 < K && dv_a + 16 < V}};
  const int e00 = dk_a * V + dv_a;
  const int eo[2][2] = {{ok[0][0] ? e00 : 0, ok[0][1] ? e00 + 16 : 0},
                        {ok[1][0] ? e00 + V : 0, ok[1][1] ? e00 + V + 16 : 0}};
  const float* pb = partial + bh * nparts * stride;
  float a[2][2] = {{0.f, 0.f}, {0.f, 0.f}};
  int pidx = 0;
  for (; pidx + 4 <= nparts; pidx += 4) {
    float x[4][2][2];
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) x[u][i][j] = pb[(int64_t)(pidx + u) * stride + eo[i][j]];
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) a[i][j] += x[u][i][j];
  }
  for (; pidx < nparts; ++pidx)
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j) a[i][j] += pb[(int64_t)pidx * stride + eo[i][j]];
  const float corr[2][2] = {{c00, c01}, {c10, c11}};
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
      if (ok[i][j]) h[bh * E + eo[i][j]] = a[i][j] - corr[i][j];
}

// Per-chunk norm of hc_c = K_c^T V_c - kc_c vc_c^T (kernel.py:172-174); partial holds one
// entry per chunk here.
__global__ __launch_bounds__(kThreads) void chunk_norm_kernel(
    const float* __restrict__ partial, const float* __restrict__ kc, const float* __restrict__ vc,
    float* __restrict__ h_norm, int K, int V, float pnorm) {
  __shared__ float red[kThreads / 64];
  const int64_t bc = blockIdx.x;
  const int E = K * V, stride = E + K;
  float acc = 0.f;
  for (int e = threadIdx.x; e < E; e += kThreads) {
    const int dk = e / V, dv = e - dk * V;
    const float x = fabsf(partial[bc * stride + e] - kc[bc * K + dk] * vc[bc * V + dv]);
    acc += pnorm == 2.f ? x * x : powf(x, pnorm);
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) acc += __shfl_xor(acc, off);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = acc;
  __syncthreads();
  if (threadIdx.x == 0) {
    const float tot = (red[0] + red[1]) + (red[2] + red[3]);
    h_norm[bc] = pnorm == 2.f ? sqrtf(tot) : powf(tot, 1.f / pnorm);
  }
}

// 16-bit pack / unpack helpers of the attention kernel
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

// (written as a vector conversion so that the compiler can use the packed conversion instruction)
template <typename T> __device__ __forceinline__ uint32_t pack_pair(float a, float b) {
  typedef float f32x2_t __attribute__((ext_vector_type(2)));
  typedef T tx2_t __attribute__((ext_vector_type(2)));
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2_t{a, b}, tx2_t));
}
template <typename T> __device__ __forceinline__ float unpack_lo(uint32_t w) {
  return (float)__builtin_bit_cast(T, (uint16_t)(w & 0xffffu));
}
template <typename T> __device__ __forceinline__ float unpack_hi(uint32_t w) {
  return (float)__builtin_bit_cast(T, (uint16_t)(w >> 16));
}

// ===========================================================================
// attention kernel
// ===========================================================================
// One workgroup (4 waves) per (head, 64-query block).  Wave w owns queries
// 32*(w%2) .. +31 and, of every 64-key block, keys 32*(w/2) .. +31: the two waves that
// share a query half keep separate running maxima / sums / accumulators for their key
// halves and are merged once at the end.  MFMA: v_mfma_f32_32x32x16 (A lane l: m = l%32,
// k = 8*(l/32)+i; B lane l: n = l%32, same k; C lane l: column l%32, register r is row
// 8*(r/4) + 4*(l/32) + r%4).
//   S^T[key][query] = K Q^T      A = K tile row (16 B of one key), B = Q^T in registers
//   O^T[vcol][query] += V^T P^T  A = eight keys of one value column, taken out of the
//                                row-major V tile by the transposing LDS read (two reads of
//                                four keys), B = exp2(S^T) packed to 16 bits, straight from the
//                                accumulator registers: k-slot i of k-step t is register
//                                8t+i, i.e. key 16t + 8*(i/4) + 4*(l/32) + i%4
//   phase 1  exact softmax attention over the NS selected 64-key blocks
//   phase 2  the unselected blocks, each represented by its mean key (weight n_c in the
//            denominator) and its value sum; means / sums are hi + lo 16-bit pairs
//   phase 3  first-order term: acc += (q H) * (G/T) * scale, q H precomputed per token
//   o = acc / (l + G)
// Unlike the Triton kernel (kernel.py:263-276) the running G is rescaled together with
// acc and l whenever the running maximum grows.
typedef float f32x16 __attribute__((ext_vector_type(16)));

typedef short i16x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2t __attribute__((ext_vector_type(2)));
// Eight keys of one value column (an MFMA operand fragment of one k-step) out of a row-major
// tile: two transposing reads of gfx950 (in a block of 16 lanes, lane i receives element i%4 of
// the 8 bytes addressed by lanes i/4, 4 + i/4, 8 + i/4, 12 + i/4); `off0` / `off1` are this lane's
// byte offsets for the first / second four keys.
__device__ __forceinline__ u32x4 tr_fragment(const unsigned char* tile, int off0, int off1) {
  typedef i16x4 __attribute__((address_space(3))) * lds_i16x4;
  const i16x4 a = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4)(tile + off0));
  const i16x4 b = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4)(tile + off1));
  const u32x2t wa = __builtin_bit_cast(u32x2t, a), wb = __builtin_bit_cast(u32x2t, b);
  return u32x4{wa[0], wa[1], wb[0], wb[1]};
}

template <typename T> struct Mma32;
template <> struct Mma32<_Float16> {
  static __device__ __forceinline__ f32x16 run(u32x4 a, u32x4 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a),
                                                  __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
};
template <> struct Mma32<__bf16> {
  static __device__ __forceinline__ f32x16 run(u32x4 a, u32x4 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                   __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
};

struct Attn32Args {
  const void *q, *k;             // [BH, T, K]
  const void* v;                 // [BH, T, V]
  const void *kc_hi, *kc_lo;     // [BH, NTp, K] chunk mean keys, hi + lo
  const void *vc_hi, *vc_lo;     // [BH, NTp, V] chunk value sums, hi + lo
  const void* r;                 // [BH, T, V] q H per token
  const int32_t* indices;        // [BH, NT, NS]
  void* o;                       // [BH, T, V]
  int T, NT, NTp, NS;            // NT blocks of `block` tokens (NTp: padded to a multiple of 64)
  int block, NTq;                // block: a multiple of 64; NTq query tiles of 64 tokens
  float scale;
};

template <int K, int V> struct Attn32Layout {
  static constexpr int kKT = 64 * K * 2;   // K tile: 64 keys x K features
  static constexpr int kVT = 64 * V * 2;   // V tile: 64 keys x V value columns
  static constexpr int kSlot = kKT > kVT ? kKT : kVT;
  static constexpr int kTiles = 3 * kSlot;  // ring of three tiles; the selected-block bitmap follows
};

typedef uint32_t u32x2p __attribute__((ext_vector_type(2)));

// Tiles are consumed as one stream: K and V^T of selected block 0, K and V^T of block 1, ...,
// then per group of 64 unselected-block statistics the mean keys (hi, lo) and the value sums
// (hi, lo).  Stage s works on tile s in ring slot s % 3 while tile s+1 has landed or is landing
// and tile s+2 is requested: three tiles of 16 KiB per workgroup instead of two K + V^T pairs,
// so that three workgroups (three waves per SIMD, at most 168 registers) share a CU.
//
// Block sizes.  A block of a multiple of 64 tokens is several key tiles in a row, and the query
// tiles of one block share its selection.  SUB = true: blocks of 16 or 32 tokens.  The 64 queries
// of the workgroup then belong to 64 / block query blocks with selections of their own: the tile
// stream of phase 1 serves them one after the other, a key tile is put together from 64 / block
// selected blocks of the query block it belongs to, and the queries of the other query blocks
// are masked (waves without a query of that block skip the tile's arithmetic, so the exact
// branch runs at block / 32 of its speed, at most 1); every query block has its own bitmap of
// selected blocks for phase 2.
template <typename T, int K, int V, bool SUB>
__global__ __launch_bounds__(kThreads, 3) void attention32_kernel(Attn32Args a) {
  using LY = Attn32Layout<K, V>;
  constexpr int KS = K / 16;                 // k-steps of the score product
  constexpr int MB = V / 32;                 // 32-row blocks of O^T
  constexpr int OLD = 64 * (V / 8) / kThreads;
  constexpr float kNegInf = -__builtin_huge_valf();
  constexpr float kLazy = 8.f;
  // Three separate LDS objects: the compiler can then tell that a tile load in flight towards
  // one slot does not touch the slot being read, and does not make the reads wait for it.
  // The selected-block bitmap is the dynamic part.
  __shared__ __attribute__((aligned(1024))) unsigned char ring0[LY::kSlot];
  __shared__ __attribute__((aligned(1024))) unsigned char ring1[LY::kSlot];
  __shared__ __attribute__((aligned(1024))) unsigned char ring2[LY::kSlot];
  extern __shared__ __attribute__((aligned(16))) unsigned char sel[];

  const int tq = blockIdx.x % a.NTq;
  const int64_t bh = blockIdx.x / a.NTq;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int qh = wave & 1, kh = wave >> 1;
  const int n = lane & 31, kg = lane >> 5;
  const int qtok = tq * 64 + 32 * qh + n;  // this lane's query
  const float c2 = a.scale * 1.44269504f;  // scores are kept unscaled; p = exp2(s*c2 - m*c2)

  const T* qb = (const T*)a.q + bh * a.T * K;
  // buffer descriptor: base, no stride, byte count (loads past it return zeros), raw 32-bit data
  typedef int i32x4s __attribute__((ext_vector_type(4)));
  auto descriptor = [](const void* base, int64_t bytes) {
    const uint64_t p = reinterpret_cast<uint64_t>(base);
    return i32x4s{__builtin_amdgcn_readfirstlane((int)(uint32_t)p),
                  __builtin_amdgcn_readfirstlane((int)((uint32_t)(p >> 32) & 0xffffu)),
                  __builtin_amdgcn_readfirstlane((int)bytes), 0x00020000};
  };
  const auto k_rs = descriptor((const T*)a.k + bh * a.T * K, (int64_t)a.T * K * 2);
  const auto v_rs = descriptor((const T*)a.v + bh * a.T * V, (int64_t)a.T * V * 2);
  const auto kch_rs = descriptor((const T*)a.kc_hi + bh * a.NTp * K, (int64_t)a.NTp * K * 2);
  const auto kcl_rs = descriptor((const T*)a.kc_lo + bh * a.NTp * K, (int64_t)a.NTp * K * 2);
  const auto vch_rs = descriptor((const T*)a.vc_hi + bh * a.NTp * V, (int64_t)a.NTp * V * 2);
  const auto vcl_rs = descriptor((const T*)a.vc_lo + bh * a.NTp * V, (int64_t)a.NTp * V * 2);

  // SUB: query blocks per query tile = selected blocks per key tile, tiles per query block
  const int lg = 31 - __builtin_clz(a.block);
  const int sub = SUB ? 64 >> lg : 1, tpj = SUB ? (a.NS + sub - 1) >> (6 - lg) : 0;
  for (int i = tid; i < sub * a.NTp; i += kThreads) sel[i] = 0;
  __syncthreads();
  // A block of `block` tokens is `tpb` tiles of 64 keys; the 64 queries of this workgroup lie in
  // query block tq / tpb and share its selection.
  const int tpb = SUB ? 1 : a.block >> 6, NE = SUB ? sub * tpj : a.NS * tpb;
  const int32_t* idx = a.indices + (bh * a.NT + (SUB ? tq * sub : tq / tpb)) * a.NS;
  // first key row and row count of every tile of the selected blocks (0 rows: an index out of
  // range, or a tile past the end of the last block), kept in
  // LDS: the stages below read them with LDS loads, which the tile loads' counter does not see
  // (the list is padded with empty tiles to a multiple of three, and one more group of three)
  int2* blk = reinterpret_cast<int2*>(sel + ((sub * a.NTp + 15) & ~15));
  // SUB: first key row of each of the tile's selected blocks, -1: none (list exhausted, index out
  // of range, or a query block past the end of the sequence)
  int4* blk4 = reinterpret_cast<int4*>(blk);
  if constexpr (SUB) {
    for (int i = tid; i < (NE + 2) / 3 * 3 + 3; i += kThreads) {
      int r0[4] = {-1, -1, -1, -1};
      const int j = i / max(tpj, 1), t = i - j * tpj;
      if (i < NE && tq * sub + j < a.NT)
        for (int pc = 0; pc < sub; ++pc) {
          const int e = t * sub + pc;
          const int b = e < a.NS ? idx[(int64_t)j * a.NS + e] : -1;
          if (b >= 0 && b < a.NT) {
            r0[pc] = b << lg;
            sel[j * a.NTp + b] = 1;
          }
        }
      blk4[i] = int4{r0[0], r0[1], r0[2], r0[3]};
    }
  } else {
    for (int i = tid; i < (NE + 2) / 3 * 3 + 3; i += kThreads) {
      const int b = i < NE ? idx[i / tpb] : -1;
      const bool ok = b >= 0 && b < a.NT;
      if (ok) sel[b] = 1;
      const int row0 = b * a.block + 64 * (i % tpb);
      blk[i] = ok && row0 < a.T ? int2{row0, min(64, a.T - row0)} : int2{0, 0};
    }
  }

  // Q^T operand: k-step s covers features 16s + 8kg + i
  u32x4 qop[KS];
#pragma unroll
  for (int s = 0; s < KS; ++s)
    qop[s] = qtok < a.T ? *reinterpret_cast<const u32x4*>(qb + (int64_t)qtok * K + 16 * s + 8 * kg)
                        : u32x4{0u, 0u, 0u, 0u};

  // 16-byte chunk ch of row `row`, XOR-swizzled (rows are 128 or 256 bytes: a column of
  // rows would otherwise sit in one bank group)
  // (the LDS serves 16 lanes x 16 bytes per cycle from 64 banks: 16 consecutive rows of a
  // column must land in 16 different 16-byte bank groups; 256-byte rows need all four low
  // row bits, 128-byte rows come in pairs that already differ in the upper half of the banks)
  auto swz256 = [](int row, int ch) { return row * 256 + ((ch ^ (row & 15)) << 4); };
  auto swz128 = [](int row, int ch) { return row * 128 + ((ch ^ ((row >> 1) & 7)) << 4); };
  auto kswz = [&](int row, int ch) { return K == 128 ? swz256(row, ch) : swz128(row, ch); };
  // V tiles are read four consecutive keys x 64 bytes at a time (transposing reads): the 64-byte
  // group of a row moves with the two low key bits (256-byte rows) / with key bit 1 (128-byte
  // rows, whose neighbours already differ in the upper half of the banks)
  auto vswz = [&](int row, int ch) {
    return V == 128 ? row * 256 + ((ch ^ ((row & 3) << 2)) << 4) : row * 128 + ((ch ^ (((row >> 1) & 1) << 2)) << 4);
  };
  auto oswz = [&](int row, int ch) { return V == 128 ? swz256(row, ch) : swz128(row, ch); };

  // Tiles go from global memory straight into LDS (buffer load with the LDS destination:
  // lane l of a wave instruction delivers 16 bytes to destination + 16*l, so one instruction
  // fills 1 KiB = 4 or 8 whole tile rows).  The swizzle is applied on the global side: the
  // lane that owns LDS slot s of row r fetches chunk s ^ swizzle(r).  Rows past the end of
  // the tensor arrive as zeros (the descriptor's byte count is the bounds check).
  // The loads are written as assembly: the compiler's own wait insertion then neither counts
  // them nor waits for all of them before the first read of a slot; the waits are the ones at
  // the start of each stage below.
  typedef __attribute__((address_space(3))) unsigned char* lds_ptr;
  auto dma16 = [](i32x4s rs, unsigned char* dst, uint32_t lane_off, int wave_off) {
    const uint32_t lds = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(lds_ptr)dst);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                 :
                 : "s"(lds), "v"(lane_off), "s"(rs), "s"(wave_off)
                 : "memory", "m0");
  };
  constexpr int KROWB = K * 2, KRW = 1024 / KROWB, KJ = 64 / (4 * KRW);
  const int krow_l = KRW * wave + lane / (KROWB / 16), kslot = lane % (KROWB / 16);
  const uint32_t k_lane_off =
      (uint32_t)(krow_l * KROWB + ((kslot ^ (K == 128 ? (krow_l & 15) : ((krow_l >> 1) & 7))) << 4));
  auto dma_tile_k = [&](i32x4s rs, unsigned char* tile, int row0) {
#pragma unroll
    for (int j = 0; j < KJ; ++j)
      dma16(rs, tile + (4 * KRW * j + KRW * wave) * KROWB, k_lane_off, (row0 + 4 * KRW * j) * KROWB);
  };
  // V tile: the same with its own row size and swizzle
  constexpr int VROWB = V * 2, VRW = 1024 / VROWB, VJ = 64 / (4 * VRW);
  const int vrow_l = VRW * wave + lane / (VROWB / 16), vslot = lane % (VROWB / 16);
  const uint32_t v_lane_off =
      (uint32_t)(vrow_l * VROWB + ((vslot ^ (V == 128 ? ((vrow_l & 3) << 2) : (((vrow_l >> 1) & 1) << 2))) << 4));
  auto dma_tile_v = [&](i32x4s rs, unsigned char* tile, int row0) {
#pragma unroll
    for (int j = 0; j < VJ; ++j)
      dma16(rs, tile + (4 * VRW * j + VRW * wave) * VROWB, v_lane_off, (row0 + 4 * VRW * j) * VROWB);
  };
  // SUB: a tile put together from up to four selected blocks (a, b, c, d: their first key rows, -1:
  // none).  The rows of one load instruction (4 or 8) lie in one block; the rows of a missing block
  // are requested past the end of the tensor and arrive as zeros.
  struct Tile { int a, b, c, d; };
  auto source_row = [&](const Tile& t, int R) {  // of tile row R
    const int pc = R >> lg;
    const int r0 = pc == 0 ? t.a : pc == 1 ? t.b : pc == 2 ? t.c : t.d;
    return r0 >= 0 ? r0 + (R & (a.block - 1)) : a.T;
  };
  auto dma_pieces_k = [&](unsigned char* tile, const Tile& t) {
#pragma unroll
    for (int j = 0; j < KJ; ++j) {
      const int R = 4 * KRW * j + KRW * wave;
      dma16(k_rs, tile + R * KROWB, k_lane_off - KRW * wave * KROWB, source_row(t, R) * KROWB);
    }
  };
  auto dma_pieces_v = [&](unsigned char* tile, const Tile& t) {
#pragma unroll
    for (int j = 0; j < VJ; ++j) {
      const int R = 4 * VRW * j + VRW * wave;
      dma16(v_rs, tile + R * VROWB, v_lane_off - VRW * wave * VROWB, source_row(t, R) * VROWB);
    }
  };

  // per-lane LDS offsets of the operand reads
  // (k-step s of the key tile sits at koff0 ^ (s << 5): the swizzle is an XOR of the chunk index)
  int koff0 = kswz(32 * kh + n, kg);
  // transposing reads of the V tile: in a block of 16 lanes, lane s addresses key
  // 32kh + 4kg + s/4 (+ 16t + 8x for k-step t, half x: immediate offsets) and the four value
  // columns 16(g&1) + 4(s%4) .. +3 of the 32-column block (g = lane/16); block mb of the 32-column
  // blocks sits at voff0 ^ (mb << 6)
  int voff0;
  {
    const int g16 = lane >> 4, s16 = lane & 15;
    const int f0 = 16 * (g16 & 1) + 4 * (s16 & 3);
    voff0 = vswz(32 * kh + 4 * kg + (s16 >> 2), f0 >> 3) + ((f0 >> 2) & 1) * 8;
  }

  const int kbase = 32 * kh + 4 * kg;
  float m_i = kNegInf, l_p = 0.f, g_p = 0.f;  // running max (unscaled); per-lane partial sums
  f32x16 acc[MB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[mb][r] = 0.f;

  // This wave's keys of a 64-key block are key(r) = kbase + c(r), kbase = 32kh + 4kg (per lane),
  // c(r) = 8(r/4) + r%4 (a constant per register): the predicates below compare kbase with a
  // scalar, so that no register holds a key index.
  // The tags are compile-time (std::true_type / false_type): masked = some keys are invalid,
  // weighted = the block statistics branch (sums weighted by chunk length).
  //   scores:   S^T += K Q^T
  //   softmax:  running maximum, p = exp2(...), partial sums, accumulator rescale; p packed
  //   values:   O^T += V^T P^T
  auto scores = [&](const unsigned char* kt, f32x16 st) {
    asm volatile("" : "+v"(koff0));  // the eight offsets are derived here, not kept in registers
#pragma unroll
    for (int s = 0; s < KS; ++s)
      st = Mma32<T>::run(*reinterpret_cast<const u32x4*>(kt + (koff0 ^ (s << 5))), qop[s], st);
    return st;
  };
  auto softmax = [&](f32x16 st, u32x4(&pw)[2], auto valid, auto weight, auto masked_tag, auto weighted_tag) {
    constexpr bool masked = decltype(masked_tag)::value, weighted = decltype(weighted_tag)::value;
    float mx = kNegInf;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      if constexpr (masked) st[r] = valid(8 * (r >> 2) + (r & 3)) ? st[r] : kNegInf;
      mx = fmaxf(mx, st[r]);
    }
    {  // maximum with the other half-wave's lane of the same query: one swap of the 32-lane halves
       // (assembly: the second result of the compiler's builtin for this instruction comes back
       // equal to the first in this toolchain; two wait states after the vector write of mx)
      float own = mx, other = mx;
      asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(own), "+v"(other));
      mx = fmaxf(own, other);
    }
    // The reference point of the exponents follows the running maximum lazily: it moves only
    // when the maximum has grown by more than kLazy binary orders, so p stays below 2^kLazy
    // (exact in fp32 sums, in range for a 16-bit operand) and the accumulators are rescaled a
    // few times per query block instead of on almost every tile (some row of the 32 sets a new
    // maximum in most tiles).  m_i = -inf: the first finite score is taken at once.
    const float m_new = ((mx - m_i) * c2 > kLazy) ? mx : m_i;
    const float m_safe = m_new == kNegInf ? 0.f : m_new;
    const float alpha = __builtin_amdgcn_exp2f((m_i - m_safe) * c2);
    const float mc = m_safe * c2;
    m_i = m_new;
    float psum = 0.f, wsum = 0.f;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int r = 8 * t + 2 * i;
        const float p0 = __builtin_amdgcn_exp2f(fmaf(st[r], c2, -mc));
        const float p1 = __builtin_amdgcn_exp2f(fmaf(st[r + 1], c2, -mc));
        psum += p0 + p1;
        if constexpr (weighted) {
          wsum = fmaf(p0, weight(8 * (r >> 2) + (r & 3)), wsum);
          wsum = fmaf(p1, weight(8 * ((r + 1) >> 2) + ((r + 1) & 3)), wsum);
        }
        pw[t][i] = pack_pair<T>(p0, p1);
      }
    if constexpr (weighted) {
      g_p = g_p * alpha + wsum;
      l_p = l_p * alpha;
    } else {
      l_p = l_p * alpha + psum;
      g_p = g_p * alpha;
    }
    if (__any(alpha != 1.f)) {  // the running maximum rarely moves after the first blocks
#pragma unroll
      for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[mb][r] *= alpha;
    }
  };
  auto values = [&](const unsigned char* vt, const u32x4(&pw)[2]) {
    asm volatile("" : "+v"(voff0));  // the offsets of the column blocks are derived here
    // every fragment is requested before the first product (the score accumulators are dead
    // here, so the registers are there): one LDS latency per stage instead of one per column block
    u32x4 av[MB][2];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      const int off = voff0 ^ (mb << 6);
#pragma unroll
      for (int t = 0; t < 2; ++t) av[mb][t] = tr_fragment(vt + 16 * t * VROWB, off, off + 8 * VROWB);
    }
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
      for (int t = 0; t < 2; ++t) acc[mb] = Mma32<T>::run(av[mb][t], pw[t], acc[mb]);
    // (scheduling groups: the reads of two column blocks, then products and the reads of the next
    // column block in turn, so that eight reads are in flight ahead of the matrix instructions;
    // the scheduler would otherwise read one column block, wait, multiply, read the next)
    __builtin_amdgcn_sched_group_barrier(0x100, 8, 0);
#pragma unroll
    for (int mb = 2; mb < MB; ++mb) {
      __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 4, 0);
    }
    __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);
  };
  const std::true_type yes{};
  const std::false_type no{};

  // ---- the tile stream ----
  // Phase 1 is padded to a multiple of three blocks (six stages) and phase 2 to a multiple of
  // three groups (twelve stages), so that the ring slot of every stage is a compile-time
  // constant in loops unrolled by that much; padding stages request and compute nothing.
  const int NS3 = (NE + 2) / 3 * 3, S1 = 2 * NS3;
  const int NG = (a.NT + 63) / 64;
  // phase 2 by stream position (s >= S1): number of load instructions a wave issues for tile s
  // (0: no such tile), and the request itself
  auto tile_loads = [&](int s) {
    const int s2 = s - S1;
    return (s2 >> 2) < NG ? ((s2 & 2) ? VJ : KJ) : 0;
  };
  auto fetch = [&](int s, unsigned char* slot) {
    const int s2 = s - S1, g = s2 >> 2;
    if (g < NG) {
      switch (s2 & 3) {
        case 0: dma_tile_k(kch_rs, slot, g * 64); break;
        case 1: dma_tile_k(kcl_rs, slot, g * 64); break;
        case 2: dma_tile_v(vch_rs, slot, g * 64); break;
        default: dma_tile_v(vcl_rs, slot, g * 64); break;
      }
    }
  };
  // Start of a stage: this wave's loads of the stage's tile have landed (the `pending` loads of
  // the next tile, issued later, may still be in flight: the counter retires in order), every
  // wave has said so and has finished reading the previous tile, whose slot is then free for
  // the tile after the next.
  auto begin_stage = [&](int pending) {
    if (pending >= 4) asm volatile("s_waitcnt vmcnt(4) lgkmcnt(0)\n\ts_barrier" ::: "memory");
    else if (pending >= 2) asm volatile("s_waitcnt vmcnt(2) lgkmcnt(0)\n\ts_barrier" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
  };
  static_assert(KJ == 2 || KJ == 4, "tile load counts are waited for as 2 or 4");
  static_assert(VJ == 2 || VJ == 4, "tile load counts are waited for as 2 or 4");

  u32x4 pw[2];
  f32x16 zero16;
#pragma unroll
  for (int r = 0; r < 16; ++r) zero16[r] = 0.f;
  const auto none = [](int) { return 0.f; };

  // ---- phase 1: the tiles of the selected blocks, three per iteration (not SUB: first key row a,
  // row count b of each; an empty tile - no such block - requests and computes nothing) ----
  auto block_info = [&](int i) {
    if constexpr (SUB) {
      const int4 v = blk4[i];
      return Tile{__builtin_amdgcn_readfirstlane(v.x), __builtin_amdgcn_readfirstlane(v.y),
                  __builtin_amdgcn_readfirstlane(v.z), __builtin_amdgcn_readfirstlane(v.w)};
    } else {
      const int2 v = blk[i];
      return Tile{__builtin_amdgcn_readfirstlane(v.x), __builtin_amdgcn_readfirstlane(v.y), 0, 0};
    }
  };
  auto has = [&](const Tile& t) {
    if constexpr (SUB) return (t.a & t.b & t.c & t.d) >= 0;
    else return t.b != 0;
  };
  auto request_k = [&](unsigned char* slot, const Tile& t) {
    if constexpr (SUB) dma_pieces_k(slot, t);
    else dma_tile_k(k_rs, slot, t.a);
  };
  auto request_v = [&](unsigned char* slot, const Tile& t) {
    if constexpr (SUB) dma_pieces_v(slot, t);
    else dma_tile_v(v_rs, slot, t.a);
  };
  // SUB: does tile i belong to a query block with queries in this wave?  (tiles come grouped by
  // query block, tpj each)
  auto owner = [&](int i) { return (i >= tpj) + (i >= 2 * tpj) + (i >= 3 * tpj); };
  auto mine = [&](const Tile& t, int i) {
    if constexpr (SUB) return has(t) && ((owner(i) << lg) >> 5) == qh;
    else return has(t);
  };
  auto key_compute = [&](const unsigned char* cur, const Tile& t, int i) {
    if constexpr (SUB) {
      if (!mine(t, i)) return;
      const f32x16 st = scores(cur, zero16);
      // this wave's 32 keys are two groups of 16 with nA / nB valid rows: two blocks of 16, or the
      // halves of a block of 32; a lane counts them only if its query lies in the tile's query block
      const int pa = (32 * kh) >> lg;
      const int ra = pa == 0 ? t.a : pa == 1 ? t.b : pa == 2 ? t.c : t.d;
      const int rb = pa == 0 ? t.b : pa == 2 ? t.d : -1;  // (blocks of 16: the wave's second block)
      const int na = ra >= 0 ? min(a.block, a.T - ra) : 0;
      const int nb = a.block == 32 ? na - 16 : (rb >= 0 ? min(16, a.T - rb) : 0);
      const bool own = ((32 * qh + n) >> lg) == owner(i);
      const int nal = own ? na : 0, nbl = own ? nb : 0;
      int kg4 = 4 * kg;
      asm volatile("" : "+v"(kg4));
      softmax(st, pw, [&](int c) { return c < 16 ? kg4 < nal - c : kg4 < nbl - (c - 16); }, none, yes, no);
    } else {
      const int nrows = t.b;
      if (nrows == 64) {
        const f32x16 st = scores(cur, zero16);
        softmax(st, pw, [](int) { return true; }, none, no, no);
      } else if (nrows > 0) {
        const f32x16 st = scores(cur, zero16);
        int kb = kbase;
        asm volatile("" : "+v"(kb));  // (keeps the sixteen sums kb + c out of registers across the loop)
        softmax(st, pw, [&](int c) { return kb < nrows - c; }, none, yes, no);
      }
    }
  };
  // the query operand has arrived before the first tile is requested: a later wait for it would
  // also wait for every tile load issued in between (the counter retires in order)
#pragma unroll
  for (int s = 0; s < KS; ++s) asm volatile("" ::"v"(qop[s]));
  __syncthreads();  // the selected blocks' rows are in LDS
  if (NS3 > 0) {
    const Tile b0 = block_info(0);
    if (has(b0)) {
      request_k(ring0, b0);
      request_v(ring1, b0);
    }
  } else {
    fetch(S1, ring0);
    fetch(S1 + 1, ring1);
  }
  for (int i0 = 0; i0 < NS3; i0 += 3) {
    const bool last = i0 + 3 == NS3;  // the tiles after this iteration's are phase 2's first two
    const Tile b0 = block_info(i0), b1 = block_info(i0 + 1), b2 = block_info(i0 + 2), b3 = block_info(i0 + 3);
    const int k3 = last ? tile_loads(S1) : (has(b3) ? KJ : 0);
    // K of b0 in slot 0
    begin_stage(has(b0) ? VJ : 0);
    if (has(b1)) request_k(ring2, b1);
    key_compute(ring0, b0, i0);
    // V of b0 in slot 1
    begin_stage(has(b1) ? KJ : 0);
    if (has(b1)) request_v(ring0, b1);
    if (mine(b0, i0)) values(ring1, pw);
    // K of b1 in slot 2
    begin_stage(has(b1) ? VJ : 0);
    if (has(b2)) request_k(ring1, b2);
    key_compute(ring2, b1, i0 + 1);
    // V of b1 in slot 0
    begin_stage(has(b2) ? KJ : 0);
    if (has(b2)) request_v(ring2, b2);
    if (mine(b1, i0 + 1)) values(ring0, pw);
    // K of b2 in slot 1
    begin_stage(has(b2) ? VJ : 0);
    if (last) fetch(S1, ring0);
    else if (has(b3)) request_k(ring0, b3);
    key_compute(ring1, b2, i0 + 2);
    // V of b2 in slot 2
    begin_stage(k3);
    if (last) fetch(S1 + 1, ring1);
    else if (has(b3)) request_v(ring1, b3);
    if (mine(b2, i0 + 2)) values(ring2, pw);
  }

  // ---- phase 2: unselected blocks through their means / sums (hi + lo 16-bit pairs) ----
  const int last_len = a.T - (a.NT - 1) * a.block;
  const float full_len = (float)a.block;
  f32x16 stw;
  auto mean_hi_stage = [&](int s, unsigned char* cur, unsigned char* slot_s2) {
    begin_stage(tile_loads(s + 1));
    fetch(s + 2, slot_s2);
    if (((s - S1) >> 2) < NG) stw = scores(cur, zero16);
  };
  auto mean_lo_stage = [&](int s, unsigned char* cur, unsigned char* slot_s2) {
    begin_stage(tile_loads(s + 1));
    fetch(s + 2, slot_s2);
    const int g = (s - S1) >> 2;
    if (g < NG) {
      const int c0 = g * 64;
      const f32x16 st = scores(cur, stw);
      int kb = kbase;
      asm volatile("" : "+v"(kb));
      // (SUB: the bitmap of this lane's query block)
      const unsigned char* selk = sel + (SUB ? ((32 * qh + n) >> lg) * a.NTp : 0) + c0 + kb;
      const int left = a.NT - c0;  // blocks from c0 on
      softmax(st, pw, [&](int c) { return kb < left - c && !selk[c]; },
              [&](int c) { return kb == left - 1 - c ? (float)last_len : full_len; }, yes, yes);
    }
  };
  auto sum_stage = [&](int s, unsigned char* cur, unsigned char* slot_s2) {
    begin_stage(tile_loads(s + 1));
    fetch(s + 2, slot_s2);
    if (((s - S1) >> 2) < NG) values(cur, pw);
  };
  for (int s = S1; s < S1 + 4 * NG; s += 12) {
    mean_hi_stage(s + 0, ring0, ring2);
    mean_lo_stage(s + 1, ring1, ring0);
    sum_stage(s + 2, ring2, ring1);
    sum_stage(s + 3, ring0, ring2);
    mean_hi_stage(s + 4, ring1, ring0);
    mean_lo_stage(s + 5, ring2, ring1);
    sum_stage(s + 6, ring0, ring2);
    sum_stage(s + 7, ring1, ring0);
    mean_hi_stage(s + 8, ring2, ring1);
    mean_lo_stage(s + 9, ring0, ring2);
    sum_stage(s + 10, ring1, ring0);
    sum_stage(s + 11, ring2, ring1);
  }
  __syncthreads();  // nothing is in flight any more (the stream has ended); the slots are free

  // ---- merge the two key halves: waves kh = 1 hand their state to waves kh = 0 ----
  float L = l_p + __shfl_xor(l_p, 32), G = g_p + __shfl_xor(g_p, 32);
  float* mrg = reinterpret_cast<float*>(qh ? ring1 : ring0);           // [value][lane]: 64 * 16 MB floats
  float* mrg3 = reinterpret_cast<float*>(ring2) + qh * 3 * 64;         // m, L, G per lane
  if (kh == 1) {
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
      for (int r = 0; r < 16; ++r) mrg[(mb * 16 + r) * 64 + lane] = acc[mb][r];
    mrg3[0 * 64 + lane] = m_i;
    mrg3[1 * 64 + lane] = L;
    mrg3[2 * 64 + lane] = G;
  }
  __syncthreads();
  if (kh == 0) {
    const float m1 = mrg3[0 * 64 + lane];
    const float m = fmaxf(m_i, m1);
    const float ms = m == kNegInf ? 0.f : m;
    const float a0 = __builtin_amdgcn_exp2f((m_i - ms) * c2), a1 = __builtin_amdgcn_exp2f((m1 - ms) * c2);
    L = L * a0 + mrg3[1 * 64 + lane] * a1;
    G = G * a0 + mrg3[2 * 64 + lane] * a1;
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[mb][r] = acc[mb][r] * a0 + mrg[(mb * 16 + r) * 64 + lane] * a1;
  }
  __syncthreads();

  // ---- phase 3 and output (waves kh = 0): acc += (q H) * (G/T) * scale, o = acc / (L + G) ----
  unsigned char* rt = ring2;  // q H tile [64][V]
  unsigned char* ot = ring0;  // output tile [64][V]
  {
    const T* rsrc = (const T*)a.r + (bh * a.T + (int64_t)tq * 64) * V;
    const int nrows = a.T - tq * 64;
#pragma unroll
    for (int j = 0; j < OLD; ++j) {
      const int qq = tid + kThreads * j, row = qq / (V / 8), ch = qq % (V / 8);
      const u32x4 x = row < nrows ? *reinterpret_cast<const u32x4*>(rsrc + (int64_t)row * V + ch * 8)
                                  : u32x4{0u, 0u, 0u, 0u};
      *reinterpret_cast<u32x4*>(rt + oswz(row, ch)) = x;
    }
  }
  __syncthreads();
  if (kh == 0) {
    const float corr = G / (float)a.T * a.scale;
    const float inv = 1.f / (L + G);
    const int qrow = 32 * qh + n;
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
      for (int r4 = 0; r4 < 4; ++r4) {
        // registers 4*r4 .. +3: value columns 32mb + 8*r4 + 4kg + 0..3 = 8 bytes of chunk 4mb + r4
        const int off = oswz(qrow, 4 * mb + r4) + 8 * kg;
        const u32x2p rw = *reinterpret_cast<const u32x2p*>(rt + off);
        const float o0 = (acc[mb][4 * r4 + 0] + unpack_lo<T>(rw[0]) * corr) * inv;
        const float o1 = (acc[mb][4 * r4 + 1] + unpack_hi<T>(rw[0]) * corr) * inv;
        const float o2 = (acc[mb][4 * r4 + 2] + unpack_lo<T>(rw[1]) * corr) * inv;
        const float o3 = (acc[mb][4 * r4 + 3] + unpack_hi<T>(rw[1]) * corr) * inv;
        *reinterpret_cast<u32x2p*>(ot + off) = u32x2p{pack_pair<T>(o0, o1), pack_pair<T>(o2, o3)};
      }
  }
  __syncthreads();
  T* ob = (T*)a.o + (bh * a.T + (int64_t)tq * 64) * V;
#pragma unroll
  for (int j = 0; j < OLD; ++j) {
    const int qq = tid + kThreads * j, row = qq / (V / 8), ch = qq % (V / 8);
    if (tq * 64 + row < a.T)
      *reinterpret_cast<u32x4*>(ob + (int64_t)row * V + ch * 8) =
          *reinterpret_cast<const u32x4*>(ot + oswz(row, ch));
  }
}

// kc (fp32 mean) / vc (fp32 sum) -> zero-padded 16-bit hi + lo arrays [BH, NTp, D]
// (one launch for both statistics: workgroups [0, wgs0) take the keys' means, the rest the values' sums)
template <typename T>
__global__ __launch_bounds__(kThreads) void split_hi_lo_kernel(const float* __restrict__ src0, T* __restrict__ hi0,
                                                               T* __restrict__ lo0, int D0,
                                                               const float* __restrict__ src1, T* __restrict__ hi1,
                                                               T* __restrict__ lo1, int D1, int64_t BH, int NT,
                                                               int NTp, int wgs0) {
  const bool second = (int)blockIdx.x >= wgs0;
  const float* __restrict__ src = second ? src1 : src0;
  T* __restrict__ hi = second ? hi1 : hi0;
  T* __restrict__ lo = second ? lo1 : lo0;
  const int D = second ? D1 : D0;
  const int64_t wg = second ? blockIdx.x - wgs0 : blockIdx.x, wgs = second ? gridDim.x - wgs0 : wgs0;
  const int64_t total = BH * NTp * D;
  for (int64_t e = wg * kThreads + threadIdx.x; e < total; e += wgs * kThreads) {
    const int d = (int)(e % D);
    const int64_t bc = e / D;
    const int c = (int)(bc % NTp);
    const int64_t bh = bc / NTp;
    float x = 0.f;
    if (c < NT) x = src[(bh * NT + c) * D + d];
    const T h = (T)x;
    hi[e] = h;
    lo[e] = (T)(x - (float)h);
  }
}

// ===========================================================================
// block selection (replaces score = qc (kc*scale)^T; torch.topk, kernel.py:304-318)
// ===========================================================================
// One workgroup per (head, kSelRows query blocks).  Scores of its rows against all NT key
// blocks are computed with fp32 FMAs out of LDS tiles (64 key blocks at a time) and kept in
// LDS; then every wave selects, for its kSelRowsPerWave rows, the NS largest scores: the threshold
// (the NS-th largest value) comes from a bitwise descent over the order-preserving integer
// image of the floats with wave-wide counts, and the selected block indices are written in
// ascending index order (ties at the threshold: lower index first).  With a bias (the
// per-block norms), log(bias + 1e-5) is added to the score: the softmax of the reference
// (kernel.py:314-315) is monotonic per row and does not change the selection.
constexpr int kSelRowsPerWave = 2, kSelRows = 4 * kSelRowsPerWave, kSelKeys = 64;

__device__ __forceinline__ uint32_t order_bits(float x) {
  const uint32_t b = __builtin_bit_cast(uint32_t, x);
  return b ^ ((b >> 31) ? 0xffffffffu : 0x80000000u);
}

// KT = 64 / 128: the head dim; KT = 0: any head dim `Kr`, staged zero-padded to a multiple of 4.
template <int KT>
__global__ __launch_bounds__(kThreads) void select_blocks_kernel(
    const float* __restrict__ qc, const float* __restrict__ kc, const float* __restrict__ bias,
    int32_t* __restrict__ indices, int NT, int NS, float scale, int Kr) {
  constexpr int RW = kSelRowsPerWave;
  const int K = KT ? KT : ((Kr + 3) & ~3);  // row length in LDS
  const int KLD = K + 4;  // padded key rows: 16-byte reads of 16 lanes hit 16 bank groups
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  float* qs = reinterpret_cast<float*>(smem);          // [kSelRows][K]
  float* kt = qs + kSelRows * K;                       // [64][K + 4]
  float* sc = kt + kSelKeys * KLD;                     // [kSelRows][NTs]
  const int NTs = (NT + 63) & ~63;
  const int nrt = (NT + kSelRows - 1) / kSelRows;
  const int r0 = (blockIdx.x % nrt) * kSelRows;
  const int64_t bh = blockIdx.x / nrt;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int Km = KT ? KT : Kr;  // row length in memory
  const float* qh = qc + bh * NT * Km;
  const float* kh = kc + bh * NT * Km;
  typedef float f4 __attribute__((ext_vector_type(4)));
  // four consecutive values of a row in memory (scalar loads and zero padding when the head dim
  // is not one of the two built-in ones)
  auto load4 = [&](const float* rowp, int c4) -> f4 {
    if constexpr (KT != 0) {
      return *reinterpret_cast<const f4*>(rowp + 4 * c4);
    } else {
      f4 x;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const bool in = 4 * c4 + i < Km;
        x[i] = rowp[in ? 4 * c4 + i : 0];
        x[i] = in ? x[i] : 0.f;
      }
      return x;
    }
  };

  for (int e = tid; e < kSelRows * (K / 4); e += kThreads) {
    const int row = e / (K / 4), c4 = e % (K / 4);
    f4 x = f4{0.f, 0.f, 0.f, 0.f};
    if (r0 + row < NT) x = load4(qh + (int64_t)(r0 + row) * Km, c4);
    *reinterpret_cast<f4*>(qs + row * K + 4 * c4) = x;
  }
  // the tile's pieces of this thread are all requested before the first is stored (clamped
  // addresses instead of branches: a loop of guarded loads waits for every single one), and the
  // next tile's while this one is multiplied
  constexpr int NPRE = KT ? kSelKeys * (KT / 4) / kThreads : kSelKeys * 32 / kThreads;
  f4 pre[NPRE];
  auto request_tile = [&](int j0) {
#pragma unroll
    for (int u = 0; u < NPRE; ++u) {
      const int e = tid + u * kThreads, row = e / (K / 4), c4 = e % (K / 4);
      const bool in = e < kSelKeys * (K / 4) && j0 + row < NT;
      pre[u] = load4(kh + (int64_t)(in ? j0 + row : 0) * Km, in ? c4 : 0);
      if (!in) pre[u] = f4{0.f, 0.f, 0.f, 0.f};
    }
  };
  request_tile(0);
  for (int j0 = 0; j0 < NT; j0 += kSelKeys) {
    __syncthreads();  // previous tile consumed (first trip: nothing to wait for but cheap)
#pragma unroll
    for (int u = 0; u < NPRE; ++u) {
      const int e = tid + u * kThreads, row = e / (K / 4), c4 = e % (K / 4);
      if (e < kSelKeys * (K / 4)) *reinterpret_cast<f4*>(kt + row * KLD + 4 * c4) = pre[u];
    }
    __syncthreads();
    if (j0 + kSelKeys < NT) request_tile(j0 + kSelKeys);
    float acc[RW];  // rows RW*wave .. +RW-1 against key j0 + lane
#pragma unroll
    for (int rr = 0; rr < RW; ++rr) acc[rr] = 0.f;
    const float* kr = kt + lane * KLD;
    const float* q0 = qs + (RW * wave) * K;
#pragma unroll 4
    for (int d = 0; d < K; d += 4) {
      const f4 kv = *reinterpret_cast<const f4*>(kr + d);
#pragma unroll
      for (int rr = 0; rr < RW; ++rr) {
        const f4 x = *reinterpret_cast<const f4*>(q0 + rr * K + d);
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[rr] = fmaf(x[i], kv[i], acc[rr]);
      }
    }
    const int key = j0 + lane;
    const float off = key < NT ? (bias ? logf(bias[bh * NT + key] + 1e-5f) : 0.f) : -__builtin_huge_valf();
#pragma unroll
    for (int rr = 0; rr < RW; ++rr) sc[(RW * wave + rr) * NTs + key] = key < NT ? acc[rr] * scale + off : off;
  }
  __syncthreads();

  // the wave's rows advance through the bitwise descent together: independent
  // chains of LDS reads and wave-wide counts instead of one
  uint32_t thr[RW];
#pragma unroll
  for (int rr = 0; rr < RW; ++rr) thr[rr] = 0u;
  for (int bit = 31; bit >= 0; --bit) {
    int cnt[RW];
#pragma unroll
    for (int rr = 0; rr < RW; ++rr) cnt[rr] = 0;
    for (int j = lane; j < NTs; j += 64)
#pragma unroll
      for (int rr = 0; rr < RW; ++rr)
        cnt[rr] += __popcll(__ballot(order_bits(sc[(RW * wave + rr) * NTs + j]) >= (thr[rr] | (1u << bit))));
#pragma unroll
    for (int rr = 0; rr < RW; ++rr)
      if (cnt[rr] >= NS) thr[rr] |= 1u << bit;
  }
#pragma unroll
  for (int rr = 0; rr < RW; ++rr) {
    const int row = RW * wave + rr;
    if (r0 + row >= NT) break;  // uniform over the wave
    const float* srow = sc + row * NTs;
    const uint32_t t = thr[rr];
    int above = 0;
    for (int j = lane; j < NTs; j += 64) above += __popcll(__ballot(order_bits(srow[j]) > t));
    int ties_left = NS - above, written = 0;
    int32_t* dst = indices + (bh * NT + (r0 + row)) * (int64_t)NS;
    for (int j = lane; j < NTs; j += 64) {
      const uint32_t u = order_bits(srow[j]);
      const uint64_t tie_mask = __ballot(u == t);
      const int tie_rank = __popcll(tie_mask & ((1ull << lane) - 1ull));
      const bool take = u > t || (u == t && tie_rank < ties_left);
      const uint64_t take_mask = __ballot(take);
      if (take) dst[written + __popcll(take_mask & ((1ull << lane) - 1ull))] = j;
      written += __popcll(take_mask);
      ties_left -= min(ties_left, (int)__popcll(tie_mask));
    }
  }
}

size_t select_blocks_lds_bytes(int NT, int K) {
  const int NTs = (NT + 63) & ~63, KP = (K + 3) & ~3;
  return (size_t)(kSelRows * KP + kSelKeys * (KP + 4) + kSelRows * NTs) * sizeof(float);
}

bool select_blocks_supported(int NT, int K) {
  return K >= 1 && K <= 128 && select_blocks_lds_bytes(NT, K) <= 160 * 1024;
}

int select_blocks(const float* qc, const float* kc, const float* bias, int32_t* indices, int64_t BH,
                  int NT, int K, int NS, float scale, hipStream_t st) {
  const int lds = (int)select_blocks_lds_bytes(NT, K);
  const int nrt = (NT + kSelRows - 1) / kSelRows;
  const dim3 grid((unsigned)(BH * nrt)), block(kThreads);
  auto run = [&](auto kernel) {
    if (lds > 64 * 1024) {
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, lds);
      if (e != hipSuccess) {
        set_error("block selection: cannot reserve %d bytes of LDS: %s", lds, hipGetErrorString(e));
        return (int)kErrLaunch;
      }
    }
    kernel<<<grid, block, lds, st>>>(qc, kc, bias, indices, NT, NS, scale, K);
    return (int)kOk;
  };
  if (K == 64) return run(select_blocks_kernel<64>);
  if (K == 128) return run(select_blocks_kernel<128>);
  return run(select_blocks_kernel<0>);
}

static Prob dense_prob(int64_t BH, int64_t T, int K, int V) {
  Prob p;
  p.cu = nullptr;
  p.perm = nullptr;
  p.chunk_base = nullptr;
  p.N = (int)BH;
  p.H = 1;
  p.L = (int)T;
  p.Lk = 0;
  p.T = BH * T;
  p.DK = K;
  p.DV = V;
  p.scale = 1.f;
  p.eps = 0.f;
  p.flags = 0;
  return p;
}

// chunk of the K^T V reduction: the block size itself when per-chunk norms are
// wanted (one partial per chunk), else whatever fills the machine
static int state_chunk_for(const Prob& p, int dtype, int chunk, bool per_chunk) {
  if (per_chunk) return chunk;
  return mfma::supported(p, dtype) ? mfma::state_chunk(p, true) : generic::state_chunk(p);
}

size_t chunk_reduce_workspace_bytes(int64_t BH, int64_t T, int K, int V, int chunk, int dtype,
                                    bool per_chunk) {
  const Prob p = dense_prob(BH, T, K, V);
  const int sc = state_chunk_for(p, dtype, chunk, per_chunk);
  const int64_t nparts = cdiv64(T, sc);
  return align_up((size_t)BH * nparts * ((size_t)K * V + K) * sizeof(float), 256);
}

template <typename T>
static void launch_sums(const void* q, const void* k, const void* v, float* qc, float* kc, float* vc,
                        int64_t BH, int Tn, int NT, int chunk, int K, int V, bool q_only, hipStream_t st) {
  if constexpr (sizeof(T) == 2) {
    if ((K == 64 || K == 128) && (q_only || V == K)) {
      const int nten = q_only ? 1 : 3;
      const dim3 grid((unsigned)cdiv64(BH * NT * nten, 4)), block(kThreads);
      if (K == 64)
        chunk_sums16_kernel<T, 64><<<grid, block, 0, st>>>((const T*)q, (const T*)k, (const T*)v, qc, kc, vc, BH, Tn, NT, chunk, nten);
      else
        chunk_sums16_kernel<T, 128><<<grid, block, 0, st>>>((const T*)q, (const T*)k, (const T*)v, qc, kc, vc, BH, Tn, NT, chunk, nten);
      return;
    }
  }
  chunk_sums_kernel<T><<<dim3((unsigned)cdiv64(BH * NT * 3, 4)), dim3(kThreads), 0, st>>>(
      (const T*)q, (const T*)k, (const T*)v, qc, kc, vc, BH, Tn, NT, chunk, K, V);
}

int chunk_reduce(const void* q, const void* k, const void* v, float* qc, float* kc, float* vc,
                 float* h, float* h_norm, void* workspace, int64_t BH, int64_t T, int K, int V,
                 int chunk, float pnorm, int dtype, hipStream_t st) {
  const Prob p = dense_prob(BH, T, K, V);
  const int NT = (int)cdiv64(T, chunk);
  const bool per_chunk = h_norm != nullptr;
  const int sc = state_chunk_for(p, dtype, chunk, per_chunk);
  const int nparts = (int)cdiv64(T, sc);
  float* partial = (float*)workspace;
  // 16-bit, head dims 64 / 128 (no padded variant of that kernel), 64-token blocks: k and v are read once, by the state kernel,
  // which also writes their block statistics; q has its own streaming pass
  const bool fused = dtype != kF32 && (K == 64 || K == 128) && (V == 64 || V == 128) && mfma::supported(p, dtype) &&
                     chunk == 64 && !per_chunk;
  if (dtype == kF16) launch_sums<_Float16>(q, k, v, qc, kc, vc, BH, (int)T, NT, chunk, K, V, fused, st);
  else if (dtype == kBF16) launch_sums<__bf16>(q, k, v, qc, kc, vc, BH, (int)T, NT, chunk, K, V, fused, st);
  else launch_sums<float>(q, k, v, qc, kc, vc, BH, (int)T, NT, chunk, K, V, false, st);
  if (fused) mfma::state_with_block_stats(p, dtype, k, v, partial, sc, nparts, kc, vc, NT, st);
  else if (mfma::supported(p, dtype)) mfma::state(p, dtype, k, v, k, partial, sc, nparts, st);
  else generic::state_partial(p, dtype, k, v, k, partial, sc, nparts, st);
  if (per_chunk)
    chunk_norm_kernel<<<dim3((unsigned)(BH * NT)), dim3(kThreads), 0, st>>>(partial, kc, vc, h_norm, K,
                                                                          V, pnorm);
  const int tiles_per_head = (int)(cdiv64(K, kHTile) * cdiv64(V, kHTile));
  finish_h_kernel<<<dim3((unsigned)(BH * tiles_per_head)), dim3(kThreads), 0, st>>>(
      partial, nparts, kc, vc, h, NT, K, V);
  return kOk;
}

bool attention_supported(int K, int V, int block, int dtype) {
  return (dtype == kF16 || dtype == kBF16) && (K == 64 || K == 128) && (V == 64 || V == 128) &&
         (block == 16 || block == 32 || (block >= 64 && block % 64 == 0));
}

static int64_t padded_chunks(int64_t T, int block) { return cdiv64(cdiv64(T, block), 64) * 64; }

// kc_hi | kc_lo | vc_hi | vc_lo | r
size_t attention_workspace_bytes(int64_t BH, int64_t T, int K, int V, int block) {
  const int64_t NTp = padded_chunks(T, block);
  return 2 * align_up((size_t)BH * NTp * K * 2, 256) + 2 * align_up((size_t)BH * NTp * V * 2, 256) +
         align_up((size_t)BH * T * V * 2, 256);
}

template <typename T, int K, int V, bool SUB>
static int launch_attention_variant(const Attn32Args& a, int64_t BH, hipStream_t st) {
  using LY = Attn32Layout<K, V>;
  // the tile ring is static; dynamic: the selected-block bitmaps and the tile list of phase 1
  const int sub = SUB ? 64 / a.block : 1;
  const int tiles = SUB ? sub * ((a.NS + sub - 1) / sub) : a.NS * (a.block / 64);
  const int lds = ((sub * a.NTp + 15) & ~15) + ((tiles + 2) / 3 * 3 + 3) * (SUB ? 16 : 8);
  auto kernel = attention32_kernel<T, K, V, SUB>;
  if (LY::kTiles + lds > 64 * 1024) {
    if (LY::kTiles + lds > 160 * 1024) {
      set_error("piecewise attention: %d key blocks need more LDS than a workgroup has", a.NT);
      return kErrUnsupported;
    }
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, lds);
    if (e != hipSuccess) {
      set_error("piecewise attention: cannot reserve %d bytes of LDS: %s", lds, hipGetErrorString(e));
      return kErrLaunch;
    }
  }
  kernel<<<dim3((unsigned)(BH * a.NTq)), dim3(kThreads), lds, st>>>(a);
  return kOk;
}

template <typename T, int K, int V>
static int launch_attention(const Attn32Args& a, int64_t BH, hipStream_t st) {
  return a.block < 64 ? launch_attention_variant<T, K, V, true>(a, BH, st)
                      : launch_attention_variant<T, K, V, false>(a, BH, st);
}

template <typename T>
static int attention_t(const void* q, const void* k, const void* v, const float* kc, const float* vc,
                       const float* h, const int32_t* indices, void* o, void* workspace, int64_t BH,
                       int64_t Tn, int K, int V, int block, int NS, float scale, int dtype, hipStream_t st) {
  const int NT = (int)cdiv64(Tn, block), NTq = (int)cdiv64(Tn, 64);
  const int64_t NTp = padded_chunks(Tn, block);
  char* ws = (char*)workspace;
  T* kc_hi = (T*)ws;
  ws += align_up((size_t)BH * NTp * K * 2, 256);
  T* kc_lo = (T*)ws;
  ws += align_up((size_t)BH * NTp * K * 2, 256);
  T* vc_hi = (T*)ws;
  ws += align_up((size_t)BH * NTp * V * 2, 256);
  T* vc_lo = (T*)ws;
  ws += align_up((size_t)BH * NTp * V * 2, 256);
  T* r = (T*)ws;
  const unsigned gk = (unsigned)std::min<int64_t>(cdiv64(BH * NTp * K, kThreads), 4096);
  const unsigned gv = (unsigned)std::min<int64_t>(cdiv64(BH * NTp * V, kThreads), 4096);
  split_hi_lo_kernel<T><<<dim3(gk + gv), dim3(kThreads), 0, st>>>(kc, kc_hi, kc_lo, K, vc, vc_hi, vc_lo, V, BH, NT,
                                                                  (int)NTp, (int)gk);
  // r_t = q_t H: the row-parallel kernel with M = H
  const Prob p = dense_prob(BH, Tn, K, V);
  mfma::RowsJob job{q, nullptr, h, V, 1, nullptr, nullptr, r};
  int rc = mfma::rows(p, dtype, job, K, V, st);
  if (rc != kOk) return rc;
  Attn32Args a{q, k, v, kc_hi, kc_lo, vc_hi, vc_lo, r, indices, o, (int)Tn, NT, (int)NTp, NS, block, NTq, scale};
  if (K == 64 && V == 64) return launch_attention<T, 64, 64>(a, BH, st);
  if (K == 64) return launch_attention<T, 64, 128>(a, BH, st);
  if (V == 64) return launch_attention<T, 128, 64>(a, BH, st);
  return launch_attention<T, 128, 128>(a, BH, st);
}

// ===========================================================================
// shape-generic attention kernel
// ===========================================================================
// Every head dim up to 128, every block size, fp16 / bf16 / fp32 inputs: what the MFMA kernel
// (16-bit, head dims 64 / 128, blocks of 16, 32 or a multiple of 64 tokens) does not cover.  Plain fp32 FMAs, correct
// everywhere and an order of magnitude slower.  One workgroup per (query block, head); the
// block's queries are handled 64 at a time: four neighbouring lanes share a query, each
// holding a quarter of the contraction index for the scores (summed with two lane exchanges)
// and a quarter of the value features for the accumulators.  Keys / values (phase 1), mean
// keys / value sums (phase 2) and the rows of H (phase 3) pass through LDS 32 at a time,
// converted to fp32; the softmax statistics are updated once per tile of 32 keys.
constexpr int kGenQ = 64, kGenTile = 32;

template <typename T> __device__ __forceinline__ float gen_load(const T* p) { return (float)*p; }

template <typename T>
__global__ __launch_bounds__(kThreads) void attention_generic_kernel(
    const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v, const float* __restrict__ kc,
    const float* __restrict__ vc, const float* __restrict__ h, const int32_t* __restrict__ indices,
    T* __restrict__ o, int Tn, int NT, int NS, int K, int V, int BT, float scale) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int KP = K + 1;                   // padded query rows: lanes of different queries hit different banks
  const int VS = (V + 3) / 4;             // value features per lane (at most 32)
  float* qs = reinterpret_cast<float*>(smem);        // [64][K + 1]
  float* kt = qs + kGenQ * KP;                        // [32][K]
  float* vt = kt + kGenTile * K;                      // [32][V]
  unsigned char* sel = reinterpret_cast<unsigned char*>(vt + kGenTile * V);  // [NT]
  const int blk = blockIdx.x % NT;
  const int64_t bh = blockIdx.x / NT;
  const int tid = threadIdx.x, qi = tid >> 2, part = tid & 3;
  const T* qh = q + bh * (int64_t)Tn * K;
  const T* kh = k + bh * (int64_t)Tn * K;
  const T* vh = v + bh * (int64_t)Tn * V;
  const float* kch = kc + bh * (int64_t)NT * K;
  const float* vch = vc + bh * (int64_t)NT * V;
  const float* hh = h + bh * (int64_t)K * V;
  const int32_t* idx = indices + (bh * NT + blk) * (int64_t)NS;
  const float sm_scale = scale * 1.44269504088896f;
  const float ninf = -__builtin_huge_valf();

  for (int i = tid; i < NT; i += kThreads) sel[i] = 0;
  __syncthreads();
  for (int i = tid; i < NS; i += kThreads) {
    const int c = idx[i];
    if (c >= 0 && c < NT) sel[c] = 1;
  }

  const int q_begin = blk * BT, q_end = min(Tn, q_begin + BT);
  for (int q0 = q_begin; q0 < q_end; q0 += kGenQ) {
    __syncthreads();  // the previous pass is done with the tiles; `sel` is complete
    for (int e = tid; e < kGenQ * K; e += kThreads) {
      const int row = e / K, d = e - row * K;
      qs[row * KP + d] = q0 + row < q_end ? gen_load(qh + (int64_t)(q0 + row) * K + d) : 0.f;
    }
    const bool active = q0 + qi < q_end;
    const float* qrow = qs + qi * KP;
    float acc[32], m = ninf, l = 0.f, g = 0.f;
#pragma unroll
    for (int e = 0; e < 32; ++e) acc[e] = 0.f;

    // one tile of up to 32 rows of (keys, values) in LDS, `n_c(j)` tokens behind row j
    // (1 in phase 1, the chunk length in phase 2; 0 = row does not take part)
    auto consume = [&](int rows, auto weight, bool linear) {
      float sc[kGenTile];
      float tmax = ninf;
#pragma unroll
      for (int j = 0; j < kGenTile; ++j) {
        float a = 0.f;
        if (j < rows) {
          for (int d = part; d < K; d += 4) a = fmaf(qrow[d], kt[j * K + d], a);
          a += __shfl_xor(a, 1);
          a += __shfl_xor(a, 2);
        }
        sc[j] = (j < rows && weight(j) > 0.f) ? a * sm_scale : ninf;
        tmax = fmaxf(tmax, sc[j]);
      }
      if (tmax == ninf) return;  // nothing in this tile for this query (the same for its four lanes)
      const float m_new = fmaxf(m, tmax);
      const float alpha = m == ninf ? 0.f : exp2f(m - m_new);
      l *= alpha;
      g *= alpha;
#pragma unroll
      for (int e = 0; e < 32; ++e) acc[e] *= alpha;
      m = m_new;
#pragma unroll
      for (int j = 0; j < kGenTile; ++j) {
        if (sc[j] == ninf) continue;
        const float pj = exp2f(sc[j] - m);
        if (linear) g += pj * weight(j);
        else l += pj;
#pragma unroll
        for (int e = 0; e < 32; ++e) {
          const int col = part * VS + e;
          if (e < VS && col < V) acc[e] = fmaf(pj, vt[j * V + col], acc[e]);
        }
      }
    };

    // ---- phase 1: the selected blocks, token by token ----
    for (int s_i = 0; s_i < NS; ++s_i) {
      const int c = idx[s_i];
      if (c < 0 || c >= NT) continue;
      const int t_lo = c * BT, t_hi = min(Tn, t_lo + BT);
      for (int t0 = t_lo; t0 < t_hi; t0 += kGenTile) {
        const int rows = min(kGenTile, t_hi - t0);
        __syncthreads();
        for (int e = tid; e < rows * K; e += kThreads) kt[e] = gen_load(kh + (int64_t)t0 * K + e);
        for (int e = tid; e < rows * V; e += kThreads) vt[e] = gen_load(vh + (int64_t)t0 * V + e);
        __syncthreads();
        if (active) consume(rows, [](int) { return 1.f; }, false);
      }
    }
    // ---- phase 2: every other block through its mean key and value sum ----
    for (int c0 = 0; c0 < NT; c0 += kGenTile) {
      const int rows = min(kGenTile, NT - c0);
      __syncthreads();
      for (int e = tid; e < rows * K; e += kThreads) kt[e] = kch[(int64_t)c0 * K + e];
      for (int e = tid; e < rows * V; e += kThreads) vt[e] = vch[(int64_t)c0 * V + e];
      __syncthreads();
      if (active)
        consume(rows, [&](int j) {
          const int c = c0 + j;
          return sel[c] ? 0.f : (float)min(BT, Tn - c * BT);
        }, true);
    }
    // ---- phase 3: first-order term (q H) * g / T * scale ----
    float r[32];
#pragma unroll
    for (int e = 0; e < 32; ++e) r[e] = 0.f;
    for (int d0 = 0; d0 < K; d0 += kGenTile) {
      const int rows = min(kGenTile, K - d0);
      __syncthreads();
      for (int e = tid; e < rows * V; e += kThreads) vt[e] = hh[(int64_t)d0 * V + e];
      __syncthreads();
      if (active)
        for (int j = 0; j < rows; ++j) {
          const float qd = qrow[d0 + j];
#pragma unroll
          for (int e = 0; e < 32; ++e) {
            const int col = part * VS + e;
            if (e < VS && col < V) r[e] = fmaf(qd, vt[j * V + col], r[e]);
          }
        }
    }
    if (active) {
      const float coeff = g * (1.0f / (float)Tn) * scale;
      const float inv = 1.0f / (l + g);
#pragma unroll
      for (int e = 0; e < 32; ++e) {
        const int col = part * VS + e;
        if (e < VS && col < V) o[(bh * Tn + (q0 + qi)) * (int64_t)V + col] = (T)((acc[e] + r[e] * coeff) * inv);
      }
    }
  }
}

static size_t attention_generic_lds(int NT, int K, int V) {
  return (size_t)(kGenQ * (K + 1) + kGenTile * K + kGenTile * V) * sizeof(float) + (size_t)((NT + 15) & ~15);
}

bool attention_generic_supported(int64_t T, int K, int V, int block, int dtype) {
  if (K < 1 || K > 128 || V < 1 || V > 128 || block < 1) return false;
  if (dtype != kF16 && dtype != kBF16 && dtype != kF32) return false;
  return attention_generic_lds((int)cdiv64(T > 0 ? T : 1, block), K, V) <= 160 * 1024;
}

template <typename T>
static int attention_generic_t(const void* q, const void* k, const void* v, const float* kc, const float* vc,
                               const float* h, const int32_t* indices, void* o, int64_t BH, int64_t Tn, int K,
                               int V, int block, int NS, float scale, hipStream_t st) {
  const int NT = (int)cdiv64(Tn, block);
  const int lds = (int)attention_generic_lds(NT, K, V);
  auto kernel = attention_generic_kernel<T>;
  if (lds > 64 * 1024) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, lds);
    if (e != hipSuccess) {
      set_error("piecewise attention: cannot reserve %d bytes of LDS: %s", lds, hipGetErrorString(e));
      return kErrLaunch;
    }
  }
  kernel<<<dim3((unsigned)(BH * NT)), dim3(kThreads), lds, st>>>((const T*)q, (const T*)k, (const T*)v, kc, vc, h,
                                                              indices, (T*)o, (int)Tn, NT, NS, K, V, block, scale);
  return kOk;
}

int attention_generic(const void* q, const void* k, const void* v, const float* kc, const float* vc,
                      const float* h, const int32_t* indices, void* o, int64_t BH, int64_t T, int K, int V,
                      int block, int NS, float scale, int dtype, hipStream_t st) {
  if (dtype == kF16)
    return attention_generic_t<_Float16>(q, k, v, kc, vc, h, indices, o, BH, T, K, V, block, NS, scale, st);
  if (dtype == kBF16)
    return attention_generic_t<__bf16>(q, k, v, kc, vc, h, indices, o, BH, T, K, V, block, NS, scale, st);
  return attention_generic_t<float>(q, k, v, kc, vc, h, indices, o, BH, T, K, V, block, NS, scale, st);
}

int attention(const void* q, const void* k, const void* v, const float* kc, const float* vc,
              const float* h, const int32_t* indices, void* o, void* workspace, int64_t BH, int64_t T,
              int K, int V, int block, int NS, float scale, int dtype, hipStream_t st) {
  if (dtype == kF16)
    return attention_t<_Float16>(q, k, v, kc, vc, h, indices, o, workspace, BH, T, K, V, block, NS, scale, dtype, st);
  return attention_t<__bf16>(q, k, v, kc, vc, h, indices, o, workspace, BH, T, K, V, block, NS, scale, dtype, st);
}

}  // namespace piecewise
}  // namespace fbla
