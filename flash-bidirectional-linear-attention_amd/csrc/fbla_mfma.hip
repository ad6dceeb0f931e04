// MFMA kernels for 16-bit inputs (fp16 / bf16).  A head is tiled into 64-wide blocks:
// head dims 64 and 128 exactly, every other multiple of 8 up to 128 as the next of the two
// with the rest of its last block as zero padding (the PAD variants of the kernels).
//
// Every wave is an independent worker: it streams its own 16- or 32-token
// sub-tiles, keeps fp32 accumulators in registers and touches LDS only through
// a wave-private staging area (plus one workgroup-shared, read-only matrix
// operand).  The main loops contain no workgroup barrier.
//
//  state_kernel      S_part = K~^T V and sum_t k_t over a token chunk.  Rows are
//                    read straight from global memory with one dword (2 features)
//                    per lane, so a half-wave reads one full 128-byte row; the
//                    token-major -> feature-major transposition MFMA needs is a
//                    v_perm_b32 on pairs of rows (no LDS).
//  rows_kernel       out_t = (x_t M) * rowscale_t + addvec: the forward output
//                    (M = S, rowscale = 1/(q.km+eps)) and both products of backward
//                    pass B (M = s dS and its transpose).  M is fp32 in memory and
//                    is fed to MFMA as a hi+lo pair of 16-bit operands after a
//                    power-of-two normalisation, so no precision is lost.
//
// MFMA used: v_mfma_f32_32x32x16_{f16,bf16}.  Operand layout (verified on
// gfx950): A lane l holds A[m=l%32][k=8*(l/32)+i], B lane l holds
// B[k=8*(l/32)+i][n=l%32], i=0..7; C register r of lane l is
// C[8*(r/4)+4*(l/32)+r%4][l%32].
#include <stdlib.h>

#include <type_traits>

#include "fbla_kernels.h"
#include "fbla_mfma_shared.h"

namespace fbla {
namespace mfma {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
// Which accesses carry the streaming hint (stream_load / stream_store), one bit per class so
// that each can be switched separately.
#ifndef FBLA_NT
#define FBLA_NT 31
#endif
constexpr int kNtStateLoad = 1, kNtRowsLoad = 2, kNtRowsStore = 4, kNtPassALoad = 8, kNtPassAStore = 16;
template <typename V, int BIT>
__device__ __forceinline__ V load_stream(const void* src) {
  return stream_load<(FBLA_NT & BIT) != 0, V>(src);
}
template <int BIT>
__device__ __forceinline__ void store_row16(void* dst, u32x4 w) {
  stream_store<(FBLA_NT & BIT) != 0>(dst, w);
}
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

constexpr int kThreads = 256;
constexpr int kWaves = 4;

// tiles in flight per wave in the rows kernel (128 x 128 heads run one 8-wave workgroup per
// CU and have the registers for a deeper queue)
#ifndef FBLA_ROWS_PF128
#define FBLA_ROWS_PF128 1
#endif
#ifndef FBLA_ROWS_PF
#define FBLA_ROWS_PF 1
#endif
// register budgets: four waves per SIMD for the 64 x 64 row kernel, three for the fused fp16 pass A
#ifndef FBLA_ROWS_OCC4
#define FBLA_ROWS_OCC4 1
#endif
#ifndef FBLA_ROWS_FAST
#define FBLA_ROWS_FAST 3
#endif
#ifndef FBLA_BWDA_NEXT_AT
#define FBLA_BWDA_NEXT_AT 1
#endif
#ifndef FBLA_BWDA_OCC3
#define FBLA_BWDA_OCC3 0
#endif

template <typename T> struct Ops;

template <> struct Ops<_Float16> {
  static __device__ __forceinline__ f32x16 mma(u32x4 a, u32x4 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a),
                                                  __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float c) {
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, a), __builtin_bit_cast(f16x2, b), c,
                                  false);
  }
  static __device__ __forceinline__ float lo(uint32_t w) {
    return (float)__builtin_bit_cast(_Float16, (uint16_t)(w & 0xffffu));
  }
  static __device__ __forceinline__ float hi(uint32_t w) {
    return (float)__builtin_bit_cast(_Float16, (uint16_t)(w >> 16));
  }
  static __device__ __forceinline__ uint32_t bits(float x) {
    return (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)x);
  }
  static constexpr uint32_t kOnes = 0x3c003c00u;  // (1.0, 1.0)
};

template <> struct Ops<__bf16> {
  static __device__ __forceinline__ f32x16 mma(u32x4 a, u32x4 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                   __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float c) {
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, a),
                                           __builtin_bit_cast(bf16x2, b), c, false);
  }
  static __device__ __forceinline__ float lo(uint32_t w) { return __builtin_bit_cast(float, w << 16); }
  static __device__ __forceinline__ float hi(uint32_t w) {
    return __builtin_bit_cast(float, w & 0xffff0000u);
  }
  static __device__ __forceinline__ uint32_t bits(float x) {
    return (uint32_t)__builtin_bit_cast(uint16_t, (__bf16)x);
  }
  static constexpr uint32_t kOnes = 0x3f803f80u;
};

// two floats rounded to T, packed (a in the low half): written as a vector conversion so that
// the compiler can use the packed / half-writing conversion instructions
template <typename T> __device__ __forceinline__ uint32_t pack2(float a, float b) {
  typedef float f32x2_t __attribute__((ext_vector_type(2)));
  typedef T tx2_t __attribute__((ext_vector_type(2)));
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2_t{a, b}, tx2_t));
}

// x of this lane + x of the lane 32 away (the other half-wave): one swap of the 32-lane halves in
// the vector unit instead of a permute through LDS and a wait for it
// (written as assembly: the second result of the compiler's builtin for this instruction comes
// back equal to the first in this toolchain; the two wait states cover a vector write of the
// operands just before)
__device__ __forceinline__ float sum_halves(float x) {
  float a = x, b = x;
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(a), "+v"(b));
  return a + b;  // lanes 0-31: a own, b the partner's; lanes 32-63 the other way round
}

// The callers' feature map phi(x) = elu(x) + 1 on a pair of 16-bit values, with the rounding steps
// of the torch expression `F.elu(x) + 1.0` on a 16-bit tensor (elu rounded to the type, then the sum
// rounded again), so that a forward that applies it on load agrees with one fed the mapped tensors.
template <typename T> __device__ __forceinline__ uint32_t phi_pair(uint32_t w) {
  const float x0 = Ops<T>::lo(w), x1 = Ops<T>::hi(w);
  const float e0 = x0 > 0.f ? x0 : __expf(x0) - 1.f, e1 = x1 > 0.f ? x1 : __expf(x1) - 1.f;
  const uint32_t e = pack2<T>(e0, e1);
  return pack2<T>(Ops<T>::lo(e) + 1.f, Ops<T>::hi(e) + 1.f);
}

typedef short i16x4 __attribute__((ext_vector_type(4)));
// Eight tokens of one feature (an MFMA operand fragment of one k-step) out of a row-major tile:
// two transposing reads, `off0` / `off1` are this lane's byte offsets for x = 0 / 1.
__device__ __forceinline__ u32x4 tr_fragment(const unsigned char* tile, int off0, int off1) {
  typedef i16x4 __attribute__((address_space(3))) * lds_ptr;
  const i16x4 a = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(tile + off0));
  const i16x4 b = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(tile + off1));
  const u32x2 wa = __builtin_bit_cast(u32x2, a), wb = __builtin_bit_cast(u32x2, b);
  return u32x4{wa[0], wa[1], wb[0], wb[1]};
}

// ===========================================================================
// state kernel
// ===========================================================================
// Lane l = (p = l%32, kb = l/32) owns features CK*p .. CK*p+CK-1 (CK = D/32) of
// eight tokens t0 + 8*kb + j.  A[c] / B[c] are the MFMA operands of feature
// column c: 8 tokens of one feature = 4 dwords.
template <int C> struct RowWords { uint32_t w[8][C / 2]; };

// Loads eight consecutive token rows of a 16-token tile.  `tile` is the wave-uniform address
// of the tile's first row, `step` the elements between consecutive token rows and `voff` the
// lane's constant offset (its half-wave's first row, 0 or 8, times step, plus its feature
// column).  No branch, no per-row address arithmetic in vector registers: the loads of the
// next step can stay in flight while the current one is multiplied.
template <typename T, int C>
__device__ __forceinline__ void load_rows(RowWords<C>& dst, const T* __restrict__ tile, uint32_t step,
                                          uint32_t voff) {
  // byte arithmetic in 32 bits on top of a uniform 64-bit base: the scalar-base + vector-offset
  // addressing form, one shared offset register for all eight rows
  const char* base = reinterpret_cast<const char*>(tile);
  const uint32_t step_b = step * (uint32_t)sizeof(T), voff_b = voff * (uint32_t)sizeof(T);
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const char* row = base + (size_t)((uint32_t)j * step_b);
    if constexpr (C == 2) {
      dst.w[j][0] = load_stream<uint32_t, kNtStateLoad>(row + voff_b);
    } else {
      u32x2 x = load_stream<u32x2, kNtStateLoad>(row + voff_b);
      dst.w[j][0] = x[0];
      dst.w[j][1] = x[1];
    }
  }
}

// The same with a bounds check per row, for chunks shorter than one tile: rows at or past
// `rows` (relative to the tile) are not read and come back as zero.
template <typename T, int C>
__device__ __forceinline__ void load_rows_checked(RowWords<C>& dst, const T* __restrict__ tile,
                                                  uint32_t step, int rel0, int col, int rows) {
#pragma unroll
  for (int j = 0; j < 8; ++j) {
#pragma unroll
    for (int c = 0; c < C / 2; ++c) dst.w[j][c] = 0u;
    if (rel0 + j < rows) {
      const uint32_t* src = reinterpret_cast<const uint32_t*>(tile + (size_t)(rel0 + j) * step + col);
#pragma unroll
      for (int c = 0; c < C / 2; ++c) dst.w[j][c] = src[c];
    }
  }
}

// zeroes the rows below `lo` (relative to the tile; rel0 = the lane's first row, 0 or 8)
template <int C>
__device__ __forceinline__ void mask_rows(RowWords<C>& r, int rel0, int lo) {
#pragma unroll
  for (int j = 0; j < 8; ++j)
#pragma unroll
    for (int c = 0; c < C / 2; ++c) r.w[j][c] = rel0 + j >= lo ? r.w[j][c] : 0u;
}

// keeps (keep = all ones) or clears (keep = 0) every word: lanes whose feature columns lie
// past the head dim (padding up to the 64-wide block) load a valid column and drop it here
template <int C>
__device__ __forceinline__ void keep_rows(RowWords<C>& r, uint32_t keep) {
#pragma unroll
  for (int j = 0; j < 8; ++j)
#pragma unroll
    for (int c = 0; c < C / 2; ++c) r.w[j][c] &= keep;
}

// token-pair packing: operand c gets feature c of tokens (2i, 2i+1) in dword i
template <int C>
__device__ __forceinline__ void transpose_rows(const RowWords<C>& src, u32x4 (&op)[C]) {
#pragma unroll
  for (int c2 = 0; c2 < C / 2; ++c2)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t a = src.w[2 * i][c2], b = src.w[2 * i + 1][c2];
      op[2 * c2][i] = __builtin_amdgcn_perm(b, a, 0x05040100u);      // low halves
      op[2 * c2 + 1][i] = __builtin_amdgcn_perm(b, a, 0x07060302u);  // high halves
    }
}

// SCALED = true is the feature view of the backward for head dims above 64:
// kn = q~, v = dO, every dO row is multiplied by 1/z_t (tokscal[row]) and split
// into hi + lo before the MFMA, and the vector part is dkm = sum_t dz_t q_t
// (dz_t = tokscal[total_rows + row]).
// STATS = true additionally writes, for every 64-token block of the sequence, the mean key
// (kc [N*H, NT, DK]) and the value sum (vc [N*H, NT, DV]): the block statistics of piecewise
// attention.  The waves then walk whole 64-token blocks (four tiles in a row) instead of
// interleaving single tiles, so that a block's sums stay inside one wave.
// PAD = true: the head dims (p.DK, p.DV, multiples of 8) are smaller than the template's
// DK, DV, which then only fix the tiling: rows are p.DK / p.DV elements long in memory, lanes
// of feature columns past the head dim contribute zeros, and the stored state has the true
// shape [p.DK][p.DV].
struct BlockStats {
  float* kc;
  float* vc;
  int NT;
};

// FMAP = true: the key rows arrive before the feature map and are mapped (phi_pair) as they are used.
template <typename T, int DK, int DV, bool SPLIT_KD, int TILES, bool SCALED, bool STATS = false, bool PAD = false,
          bool FMAP = false>
__global__ __launch_bounds__(kThreads, (DK == 64 && DV == 64 && !SCALED) ? 3 : 2) void state_kernel(Prob p, const T* __restrict__ kn,
                                                         const T* __restrict__ v,
                                                         const T* __restrict__ kd,
                                                         float* __restrict__ partial,
                                                         const float* __restrict__ tokscal,
                                                         int64_t total_rows, float* fin_mat,
                                                         float* fin_vec, int chunk, int nchunks,
                                                         BlockStats stats) {
  static_assert(!STATS || (TILES == 1 && !SCALED && !SPLIT_KD && !PAD), "block statistics: plain variant only");
  static_assert(!FMAP || (!SCALED && !SPLIT_KD && !PAD && !STATS), "feature map on load: plain variant only");
  const int dk = PAD ? p.DK : DK, dv = PAD ? p.DV : DV;  // row lengths in memory
  // The state is tiled into 64 x 64 blocks (64 accumulator registers per lane); a block is
  // owned by G waves that take interleaved token tiles.  For a 128 x 128 state the four
  // waves of the workgroup therefore read the same tokens, each the 64 key and 64 value
  // columns of its block: every row is fetched from HBM once and served to two waves by
  // the cache.
  constexpr int KB = DK / 64, VB = DV / 64, NB = KB * VB, G = kWaves / NB;
  constexpr int CK = 2, CV = 2;
  __shared__ float red[G > 1 ? NB * 64 * 66 : 1];  // per-group reduction buffers, [value][lane]

  __shared__ int lpt_lens[kLptMax + 1];
  const int wg_item = packed_item(p, blockIdx.x, p.H * nchunks);
  const int wg_nh = wg_item / nchunks, c = wg_item - wg_nh * nchunks;
  const int h = wg_nh % p.H;
  const int n = lpt_sequence(p, wg_nh / p.H, lpt_lens);
  const int nh = n * p.H + h;
  int64_t bos, row0, rstride;
  int len;
  seq_range(p, n, bos, len);
  // Interleaved walk (dense tensors): the nchunks workgroups of a head sweep it together,
  // workgroup c taking every nchunks-th step of kStep * G tokens, so that at any time they read
  // one moving window of the head instead of nchunks distant streams.
  constexpr int kStep = 16 * TILES;
  const bool il = !STATS && (p.flags & kInterleave) != 0;
  const int t_begin = il ? c * (kStep * G) : c * chunk;
  if (t_begin >= len) {
    if (fin_mat && c == 0) {  // empty sequence: its state is zero
      for (int e = threadIdx.x; e < dk * dv; e += kThreads) fin_mat[(int64_t)nh * dk * dv + e] = 0.f;
      if (fin_vec)
        for (int e = threadIdx.x; e < dk; e += kThreads) fin_vec[(int64_t)nh * dk + e] = 0.f;
    }
    return;
  }
  const int t_end = il ? len : min(len, t_begin + chunk);
  const int t_stride = kStep * G * (il ? nchunks : 1);
  row_base(p, n, h, bos, row0, rstride);

  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int pp = lane & 31, kb = lane >> 5;
  const int blk = wave / G, g = wave % G, bk = blk / VB, bv = blk % VB;
  // this lane's feature columns inside its block, and whether they exist
  const bool k_ok = !PAD || 64 * bk + CK * pp < dk, v_ok = !PAD || 64 * bv + CV * pp < dv;
  const int kcol0 = k_ok ? CK * pp : 0, vcol0 = v_ok ? CV * pp : 0;
  const uint32_t k_keep = k_ok ? ~0u : 0u, v_keep = v_ok ? ~0u : 0u;
  const T* kcol = kn + 64 * bk;
  const T* vcol = v + 64 * bv;
  const T* kdcol = kd + 64 * bk;

  f32x16 acc[CK][CV];
#pragma unroll
  for (int a = 0; a < CK; ++a)
#pragma unroll
    for (int b = 0; b < CV; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.f;
  float ks[CK];
#pragma unroll
  for (int a = 0; a < CK; ++a) ks[a] = 0.f;
  float kcs[CK] = {0.f, 0.f}, vcs[CV] = {0.f, 0.f};  // STATS: sums over the current 64-token block

  // Each wave walks TILES consecutive 16-token tiles per step, the steps of the G waves
  // interleaved.  Two register buffers alternate (the loop is unrolled by two so that no
  // copy is needed): the loads of the next step are issued, unconditionally, before the
  // current step is multiplied.
  struct Buf {
    RowWords<CK> k[TILES];
    RowWords<CV> v[TILES];
    RowWords<CK> d[SPLIT_KD ? TILES : 1];
    float rz[SCALED ? TILES : 1][8], dz[SCALED ? TILES : 1][8];
  };
  // A tile that would cross the end of the chunk is moved back so that it ends there; its
  // first `lo` rows were already part of the previous tile and are zeroed before use.  Every
  // tile therefore reads 16 valid rows with the same address pattern (chunks shorter than
  // one tile take the checked path below).
  const uint32_t kstep = (uint32_t)(rstride * dk), vstep = (uint32_t)(rstride * dv);
  const uint32_t kvoff = (uint32_t)(8 * kb) * kstep + (uint32_t)kcol0;
  const uint32_t vvoff = (uint32_t)(8 * kb) * vstep + (uint32_t)vcol0;
  const uint32_t tvoff = (uint32_t)(8 * kb) * (uint32_t)rstride;
  auto fetch = [&](Buf& b, int tok) {
#pragma unroll
    for (int u = 0; u < TILES; ++u) {
      const int tb = min(tok + 16 * u, t_end - 16);
      const int64_t row = row0 + (int64_t)tb * rstride;
      load_rows<T, CK>(b.k[u], kcol + row * dk, kstep, kvoff);
      load_rows<T, CV>(b.v[u], vcol + row * dv, vstep, vvoff);
      if constexpr (SPLIT_KD) load_rows<T, CK>(b.d[u], kdcol + row * dk, kstep, kvoff);
      if constexpr (SCALED) {
        const float* ts = tokscal + row;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          b.rz[u][j] = ts[tvoff + (uint32_t)j * (uint32_t)rstride];
          b.dz[u][j] = ts[total_rows + tvoff + (uint32_t)j * (uint32_t)rstride];
        }
      }
    }
  };
  auto fetch_checked = [&](Buf& b, int tok) {  // chunk shorter than a tile
#pragma unroll
    for (int u = 0; u < TILES; ++u) {
      const int rows = t_end - (tok + 16 * u);
      const int64_t row = row0 + (int64_t)(tok + 16 * u) * rstride;
      load_rows_checked<T, CK>(b.k[u], kcol + row * dk, kstep, 8 * kb, kcol0, rows);
      load_rows_checked<T, CV>(b.v[u], vcol + row * dv, vstep, 8 * kb, vcol0, rows);
      if constexpr (SPLIT_KD) load_rows_checked<T, CK>(b.d[u], kdcol + row * dk, kstep, 8 * kb, kcol0, rows);
      if constexpr (SCALED) {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const bool ok = 8 * kb + j < rows;
          b.rz[u][j] = ok ? tokscal[row + (8 * kb + j) * rstride] : 0.f;
          b.dz[u][j] = ok ? tokscal[total_rows + row + (8 * kb + j) * rstride] : 0.f;
        }
      }
    }
  };
  auto compute = [&](Buf& b, int tok, bool checked) {
    if constexpr (FMAP) {  // before any masking: phi(0) = 1, and rows that do not exist must stay zero
#pragma unroll
      for (int u = 0; u < TILES; ++u) {
        const int rows = checked ? t_end - (tok + 16 * u) : 16;
#pragma unroll
        for (int j = 0; j < 8; ++j)
#pragma unroll
          for (int c2 = 0; c2 < CK / 2; ++c2)
            b.k[u].w[j][c2] = 8 * kb + j < rows ? phi_pair<T>(b.k[u].w[j][c2]) : 0u;
      }
    }
    if constexpr (PAD) {
#pragma unroll
      for (int u = 0; u < TILES; ++u) {
        keep_rows<CK>(b.k[u], k_keep);
        keep_rows<CV>(b.v[u], v_keep);
        if constexpr (SPLIT_KD) keep_rows<CK>(b.d[u], k_keep);
      }
    }
    if (!checked && tok + kStep > t_end) {  // last step of the chunk: some tiles were moved back
#pragma unroll
      for (int u = 0; u < TILES; ++u) {
        const int lo = min(16, tok + 16 * u - min(tok + 16 * u, t_end - 16));
        mask_rows<CK>(b.k[u], 8 * kb, lo);
        if constexpr (STATS) mask_rows<CV>(b.v[u], 8 * kb, lo);
        if constexpr (SPLIT_KD) mask_rows<CK>(b.d[u], 8 * kb, lo);
        if constexpr (SCALED) {
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            b.rz[u][j] = 8 * kb + j >= lo ? b.rz[u][j] : 0.f;
            b.dz[u][j] = 8 * kb + j >= lo ? b.dz[u][j] : 0.f;
          }
        }
      }
    }
#pragma unroll
    for (int u = 0; u < TILES; ++u) {
      u32x4 A[CK], B[CV];
      transpose_rows<CK>(b.k[u], A);
      if constexpr (SCALED) {
        RowWords<CV> vh, vl;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const float rz = b.rz[u][j], dz = b.dz[u][j];
#pragma unroll
          for (int c2 = 0; c2 < CV / 2; ++c2) {
            const uint32_t w = b.v[u].w[j][c2];
            const float x0 = Ops<T>::lo(w) * rz, x1 = Ops<T>::hi(w) * rz;
            const T h0 = (T)x0, h1 = (T)x1;
            vh.w[j][c2] = pack2<T>((float)h0, (float)h1);
            vl.w[j][c2] = pack2<T>(x0 - (float)h0, x1 - (float)h1);
          }
#pragma unroll
          for (int c2 = 0; c2 < CK / 2; ++c2) {
            const uint32_t w = SPLIT_KD ? b.d[u].w[j][c2] : b.k[u].w[j][c2];
            ks[2 * c2] = fmaf(dz, Ops<T>::lo(w), ks[2 * c2]);
            ks[2 * c2 + 1] = fmaf(dz, Ops<T>::hi(w), ks[2 * c2 + 1]);
          }
        }
        u32x4 Bl[CV];
        transpose_rows<CV>(vh, B);
        transpose_rows<CV>(vl, Bl);
#pragma unroll
        for (int a = 0; a < CK; ++a)
#pragma unroll
          for (int bb = 0; bb < CV; ++bb) {
            acc[a][bb] = Ops<T>::mma(A[a], B[bb], acc[a][bb]);
            acc[a][bb] = Ops<T>::mma(A[a], Bl[bb], acc[a][bb]);
          }
      } else {
        transpose_rows<CV>(b.v[u], B);
#pragma unroll
        for (int a = 0; a < CK; ++a)
#pragma unroll
          for (int bb = 0; bb < CV; ++bb) acc[a][bb] = Ops<T>::mma(A[a], B[bb], acc[a][bb]);
        if constexpr (SPLIT_KD) {
          u32x4 Dd[CK];
          transpose_rows<CK>(b.d[u], Dd);
#pragma unroll
          for (int a = 0; a < CK; ++a)
#pragma unroll
            for (int i = 0; i < 4; ++i) ks[a] = Ops<T>::dot2(Dd[a][i], Ops<T>::kOnes, ks[a]);
        } else if constexpr (STATS) {
#pragma unroll
          for (int a = 0; a < CK; ++a) {
            float tk = 0.f;
#pragma unroll
            for (int i = 0; i < 4; ++i) tk = Ops<T>::dot2(A[a][i], Ops<T>::kOnes, tk);
            ks[a] += tk;
            kcs[a] += tk;
          }
#pragma unroll
          for (int bb = 0; bb < CV; ++bb)
#pragma unroll
            for (int i = 0; i < 4; ++i) vcs[bb] = Ops<T>::dot2(B[bb][i], Ops<T>::kOnes, vcs[bb]);
        } else {
#pragma unroll
          for (int a = 0; a < CK; ++a)
#pragma unroll
            for (int i = 0; i < 4; ++i) ks[a] = Ops<T>::dot2(A[a][i], Ops<T>::kOnes, ks[a]);
        }
      }
    }
    if constexpr (STATS) {
      // last tile of its 64-token block (or of the sequence): write the block's statistics
      if (((tok + 16) & 63) == 0 || tok + 16 >= t_end) {
        const int cb = tok >> 6;
        const float inv_n = 1.0f / (float)min(64, len - 64 * cb);
        const int64_t slot = (int64_t)nh * stats.NT + cb;
#pragma unroll
        for (int a = 0; a < CK; ++a) {
          const float tot = kcs[a] + __shfl_xor(kcs[a], 32);
          if (kb == 0 && bv == 0) stats.kc[slot * DK + 64 * bk + CK * pp + a] = tot * inv_n;
          kcs[a] = 0.f;
        }
#pragma unroll
        for (int bb = 0; bb < CV; ++bb) {
          const float tot = vcs[bb] + __shfl_xor(vcs[bb], 32);
          if (kb == 0 && bk == 0) stats.vc[slot * DV + 64 * bv + CV * pp + bb] = tot;
          vcs[bb] = 0.f;
        }
      }
    }
  };
  // token walk: single tiles interleaved over the G waves, or (STATS) whole 64-token blocks
  auto next = [&](int t) {
    if constexpr (STATS) return ((t + 16) & 63) ? t + 16 : t + 16 + 64 * (G - 1);
    else return t + t_stride;
  };
  int t0 = t_begin + (STATS ? 64 : kStep) * g;
  // fewer rows than one tile: in the interleaved walk a moved-back tile may reach into the
  // steps of other workgroups (it zeroes what it shares), so only the sequence length matters
  if (il ? len < 16 : t_end - t_begin < 16) {
    if (t0 < t_end) {
      Buf b0;
      fetch_checked(b0, t0);
      compute(b0, t0, true);
    }
  } else if (t0 < t_end) {
    Buf b0, b1;
    fetch(b0, t0);
    while (true) {
      int tn = next(t0);
      fetch(b1, tn);
      compute(b0, t0, false);
      t0 = tn;
      if (t0 >= t_end) break;
      tn = next(t0);
      fetch(b0, tn);
      compute(b1, t0, false);
      t0 = tn;
      if (t0 >= t_end) break;
    }
  }

  // one chunk per (sequence, head): the sum is final, store it scaled where the reduce
  // kernel would have put it; otherwise store this chunk's partial
  float* mat = fin_mat ? fin_mat + (int64_t)nh * dk * dv
                       : partial + partial_slot(p, n, h, c, nchunks) * (dk * dv + dk);
  float* vec = fin_mat ? (fin_vec ? fin_vec + (int64_t)nh * dk : nullptr) : mat + dk * dv;
  const float mscale = fin_mat ? seq_scale(p, len) : 1.f;
  const float vscale = fin_mat ? 1.0f / (float)len : 1.f;
  reduce_store_block<G>(acc, ks, red + (G > 1 ? blk * 64 * 66 : 0), mat + (64 * bk) * dv + 64 * bv, dv,
                        (vec && bv == 0) ? vec + 64 * bk : nullptr, mscale, vscale, g, lane,
                        PAD ? dk - 64 * bk : 64, PAD ? dv - 64 * bv : 64);
}

// ===========================================================================
// state kernel for heads tiled 128 x 128 (plain operator: no rotary keys, no row scaling,
// no block statistics)
// ===========================================================================
// A workgroup of four waves walks its chunk in steps of 64 tokens.  The rows of a step arrive
// flat (16 bytes per lane, whole rows, each read from memory exactly once) and are staged in
// LDS; wave w owns the 64 x 64 block w of the state and reads k^T and v for it straight out of
// the row-major tiles in operand order with the transposing LDS read (ds_read_b64_tr_b16), so
// nothing is transposed in registers and no wave's sum has to be added to another's at the
// end.  Two LDS buffers alternate: the step after the current one sits in registers while the
// current one is multiplied, and one barrier per step separates the writers of a buffer from
// its readers.  The contraction index is the permutation of a tile's tokens that
// bwd_a128_kernel uses (k-step ks, half-wave kb, element e = 4x + j is token 16ks + 4j + 2kb + x).
struct State128Layout {
  static constexpr int kTile = 32 * 256;     // 32 tokens x 128 features x 2 bytes
  static constexpr int kStep = 2 * kTile;    // 64 tokens
  static constexpr int kK = 0;               // k steps [2]
  static constexpr int kV = 2 * kStep;       // v steps [2]
  static constexpr int kLpt = 4 * kStep;
  static constexpr int kTotal = kLpt + (kLptMax + 1) * 4;
};

// STATS = true additionally writes the mean key and the value sum of every 64-token block (a
// step of this kernel), like state_kernel's STATS.
template <typename T, bool PAD, bool STATS = false>
__global__ __launch_bounds__(kThreads, 2) void state128_kernel(Prob p, const T* __restrict__ kn,
                                                               const T* __restrict__ v,
                                                               float* __restrict__ partial,
                                                               float* __restrict__ fin_mat,
                                                               float* __restrict__ fin_vec, int chunk,
                                                               int nchunks, BlockStats stats) {
  static_assert(!STATS || !PAD, "block statistics: full head dims only");
  using LY = State128Layout;
  constexpr int ROWB = 256;
  const int dk = PAD ? p.DK : 128, dv = PAD ? p.DV : 128;  // row lengths in memory
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int wg_item = packed_item(p, blockIdx.x, p.H * nchunks);
  const int wg_nh = wg_item / nchunks, c = wg_item - wg_nh * nchunks;
  const int h = wg_nh % p.H;
  const int n = lpt_sequence(p, wg_nh / p.H, reinterpret_cast<int*>(smem + LY::kLpt));
  const int nh = n * p.H + h;
  int64_t bos, row0, rstride;
  int len;
  seq_range(p, n, bos, len);
  const int t_begin = c * chunk;
  if (t_begin >= len) {
    if (fin_mat && c == 0) {  // empty sequence: its state is zero
      for (int e = threadIdx.x; e < dk * dv; e += kThreads) fin_mat[(int64_t)nh * dk * dv + e] = 0.f;
      if (fin_vec)
        for (int e = threadIdx.x; e < dk; e += kThreads) fin_vec[(int64_t)nh * dk + e] = 0.f;
    }
    return;
  }
  const int t_end = min(len, t_begin + chunk);
  row_base(p, n, h, bos, row0, rstride);

  const int tid = threadIdx.x, blk = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int ntok = lane & 31, kb = lane >> 5;
  const int bk = blk >> 1, bv = blk & 1;  // block (bk, bv) of the state
  unsigned char* ksteps = smem + LY::kK;
  unsigned char* vsteps = smem + LY::kV;

  // The workgroup moves the 1024 16-byte pieces of a step's 64 rows: thread t takes pieces
  // t + 256 i, i.e. chunk t % 16 of rows t / 16 + 16 i: the step's uniform address plus a uniform
  // i-th distance plus the lane's one constant byte offset (32 bits: the host keeps packed
  // tensors with more than 65536 heads away from this kernel).  Rows past the end of the chunk
  // and chunks past the head dim are not read and count as zeros.
  const int prow = tid >> 4, pch = tid & 15;
  const uint32_t krow_b = (uint32_t)rstride * (uint32_t)dk * 2u, vrow_b = (uint32_t)rstride * (uint32_t)dv * 2u;
  const uint32_t kvoff = (uint32_t)prow * krow_b + (uint32_t)pch * 16u;
  const uint32_t vvoff = PAD ? (uint32_t)prow * vrow_b + (uint32_t)pch * 16u : kvoff;
  const bool k_piece = !PAD || pch * 8 < dk, v_piece = !PAD || pch * 8 < dv;
  auto load_step = [&](u32x4(&dst)[4], const T* src, int tok0, int rowlen, uint32_t row_b, uint32_t voff, bool has) {
    const char* tp = reinterpret_cast<const char*>(src) + ((row0 + (int64_t)tok0 * rstride) * rowlen) * (int64_t)sizeof(T);
    const int rows = t_end - tok0;  // rows of this step that exist (may be <= 0)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      dst[i] = u32x4{0u, 0u, 0u, 0u};
      if (has && prow + 16 * i < rows) dst[i] = load_stream<u32x4, kNtStateLoad>(tp + (size_t)(16 * i) * row_b + voff);
    }
  };
  auto stash_step = [&](const u32x4(&src)[4], unsigned char* tiles) {
#pragma unroll
    for (int i = 0; i < 4; ++i) *reinterpret_cast<u32x4*>(tiles + swz<ROWB>(prow + 16 * i, pch)) = src[i];
  };

  f32x16 acc[2][2];
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.f;
  float ks = 0.f;  // row 64 bk + 32 bv + ntok of sum_t k_t, this half-wave's tokens

  // transposing reads: this lane addresses, for element half x, token 4 (s >> 2) + 2 (g >> 1) + x
  // (+ 16 ks) and the four features 16 (g & 1) + 4 (s & 3) .. + 3 of the fragment (g = lane / 16,
  // s = lane % 16)
  int koff[2][2], voff2[2][2];
  {
    const int g16 = lane >> 4, s16 = lane & 15;
#pragma unroll
    for (int x = 0; x < 2; ++x) {
      const int tok = 4 * (s16 >> 2) + 2 * (g16 >> 1) + x;
      const int f0 = 16 * (g16 & 1) + 4 * (s16 & 3);
#pragma unroll
      for (int a = 0; a < 2; ++a) {
        const int fk = 64 * bk + 32 * a + f0, fv = 64 * bv + 32 * a + f0;
        koff[a][x] = swz<ROWB>(tok, fk >> 3) + ((fk >> 2) & 1) * 8;
        voff2[a][x] = swz<ROWB>(tok, fv >> 3) + ((fv >> 2) & 1) * 8;
      }
    }
  }

  u32x4 rk[4], rv[4];
  load_step(rk, kn, t_begin, dk, krow_b, kvoff, k_piece);
  load_step(rv, v, t_begin, dv, vrow_b, vvoff, v_piece);
  int buf = 0;
  for (int base = t_begin; base < t_end; base += 64) {
    unsigned char* kt = ksteps + buf * LY::kStep;
    unsigned char* vt = vsteps + buf * LY::kStep;
    stash_step(rk, kt);
    stash_step(rv, vt);
    load_step(rk, kn, base + 64, dk, krow_b, kvoff, k_piece);
    load_step(rv, v, base + 64, dv, vrow_b, vvoff, v_piece);
    __syncthreads();  // the step is in LDS; every wave is done with the other buffer's previous step
    float kstep = 0.f, vstep = 0.f;  // this step's sums (STATS: the step is a block of the statistics)
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        const int tb = t * LY::kTile + s * 16 * ROWB;
        u32x4 A[2], B[2];
#pragma unroll
        for (int a = 0; a < 2; ++a) {
          A[a] = tr_fragment(kt + tb, koff[a][0], koff[a][1]);
          B[a] = tr_fragment(vt + tb, voff2[a][0], voff2[a][1]);
        }
#pragma unroll
        for (int a = 0; a < 2; ++a)
#pragma unroll
          for (int b = 0; b < 2; ++b) acc[a][b] = Ops<T>::mma(A[a], B[b], acc[a][b]);
        // sum_t k_t for the rows of A[bv] (the two waves of a key half share its 64 rows)
        const u32x4 Ak = bv ? A[1] : A[0];
#pragma unroll
        for (int i = 0; i < 4; ++i) kstep = Ops<T>::dot2(Ak[i], Ops<T>::kOnes, kstep);
        if constexpr (STATS) {  // likewise sum_t v_t for the columns of B[bk]
          const u32x4 Bv = bk ? B[1] : B[0];
#pragma unroll
          for (int i = 0; i < 4; ++i) vstep = Ops<T>::dot2(Bv[i], Ops<T>::kOnes, vstep);
        }
      }
    ks += kstep;
    if constexpr (STATS) {
      const int cb = base >> 6;
      const float inv_n = 1.0f / (float)min(64, len - 64 * cb);
      const int64_t slot = ((int64_t)nh * stats.NT + cb) * 128;
      const float totk = kstep + __shfl_xor(kstep, 32), totv = vstep + __shfl_xor(vstep, 32);
      if (kb == 0) {
        stats.kc[slot + 64 * bk + 32 * bv + ntok] = totk * inv_n;
        stats.vc[slot + 64 * bv + 32 * bk + ntok] = totv;
      }
    }
    buf ^= 1;
  }

  // one chunk per (sequence, head): the sum is final and is stored scaled where the reduce
  // kernel would have put it; otherwise this chunk's partial is stored
  float* mat = fin_mat ? fin_mat + (int64_t)nh * dk * dv
                       : partial + partial_slot(p, n, h, c, nchunks) * (dk * dv + dk);
  float* vec = fin_mat ? (fin_vec ? fin_vec + (int64_t)nh * dk : nullptr) : mat + dk * dv;
  const float mscale = fin_mat ? seq_scale(p, len) : 1.f;
  const float vscale = fin_mat ? 1.0f / (float)len : 1.f;
  float none[2] = {0.f, 0.f};
  reduce_store_block<1, false>(acc, none, nullptr, mat + (64 * bk) * dv + 64 * bv, dv, nullptr, mscale, vscale, 0,
                               lane, dk - 64 * bk, dv - 64 * bv);
  const float tot = ks + __shfl_xor(ks, 32);
  const int row = 64 * bk + 32 * bv + ntok;
  if (vec && kb == 0 && row < dk) vec[row] = tot * vscale;
}

// ===========================================================================
// rows kernel: out_t = (x_t M) * rowscale_t + addvec
// ===========================================================================
// LDS layout of a DR x DC matrix operand M: fragment f = (b*KS + s)*2 + hl holds,
// for lane l = (m = l%32, kb = l/32), the 8 values  M[(DR/2)*kb + 8s + i][sigma(b,m)]
// where sigma(b, m = 8g + 4kb' + j) = (DC/2)*kb' + 16b + 4g + j, so that after the
// MFMA every lane (token, kb') owns DC/2 consecutive output features.  M is first
// multiplied by a power of two that brings max|M| into [8,16), then split into a
// 16-bit hi part and a 16-bit lo remainder (two MFMAs recover ~fp32 accuracy).
// Returns the factor that undoes the normalisation.  Contains workgroup barriers;
// the caller must __syncthreads() before reading the fragments.
// `mat` may be the first of `nsum` partial matrices lying `sum_stride` floats apart
// (the per-chunk partials of a reduction): they are added in index order and the
// sum is multiplied by `mscale`; when `mat_out` is given the reduced matrix is
// also written there in memory order.
// PAD = true: the matrix in memory is dr x dc (multiples of 8, at most DR x DC); the
// operand's remaining rows and columns are zero.
// PAIR = true (DR = DC = 64): the matrix in memory is 32 x 32 and the operand is
// blockdiag(M, M): a 64-wide row then holds two independent 32-wide rows.
template <typename T, int DR, int DC, int NT = kThreads, bool PAD = false, bool PAIR = false>
__device__ __forceinline__ float build_operand(unsigned char* lds_opnd, float* lds_max,
                                               const float* __restrict__ mat, int ld_r, int ld_c,
                                               int nsum = 1, int64_t sum_stride = 0,
                                               float mscale = 1.f, float* mat_out = nullptr,
                                               int dr = DR, int dc = DC) {
  constexpr int KS = DR / 16;
  constexpr int kUnits = DR * DC / (8 * NT);  // units per thread
  typedef float f32x4 __attribute__((ext_vector_type(4)));
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  // A unit is eight consecutive rows r = 8*rg .. 8*rg+7 of one column cc: the eight values of
  // one lane of one fragment, i.e. one 16-byte LDS write each for the hi and the lo part.
  // Consecutive threads take consecutive memory: neighbouring columns when the column index
  // runs fastest in memory (index r*dc + cc), neighbouring row groups otherwise (cc*dr + r).
  const bool c_fast = ld_c == 1;
  float vals[kUnits][8];
  int first[kUnits];  // memory index of the unit's first element, -1 for padding
#pragma unroll
  for (int i = 0; i < kUnits; ++i) {
    const int u = tid + NT * i;
    const int rg = c_fast ? u / DC : u % (DR / 8), cc = c_fast ? u % DC : u / (DR / 8);
    if constexpr (PAIR) {
      const int r8 = 8 * (rg % 4), c32 = cc % 32;
      first[i] = (rg / 4 != cc / 32) ? -1 : (c_fast ? r8 * 32 + c32 : c32 * 32 + r8);
    } else {
      first[i] = (PAD && (8 * rg >= dr || cc >= dc)) ? -1 : (c_fast ? 8 * rg * dc + cc : cc * dr + 8 * rg);
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) vals[i][j] = 0.f;
  }
  constexpr bool kHoles = PAD || PAIR;  // some units are not backed by memory
  const int rstep = c_fast ? (PAIR ? 32 : dc) : 1;  // memory distance of consecutive rows
  for (int c = 0; c < nsum; ++c) {
    const float* src = mat + (int64_t)c * sum_stride;
    // A unit without memory behind it reads the matrix's first unit and drops it, and the choice
    // of the memory order is made outside the loops over the units: no branch between the units,
    // so the loads of all of them are in flight together.
    if (c_fast) {
#pragma unroll
      for (int i = 0; i < kUnits; ++i) {
        const bool hole = kHoles && first[i] < 0;
        const int f0 = hole ? 0 : first[i];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const float x = src[f0 + j * rstep];
          vals[i][j] += hole ? 0.f : x;
        }
      }
    } else {
#pragma unroll
      for (int i = 0; i < kUnits; ++i) {
        const bool hole = kHoles && first[i] < 0;
        const int f0 = hole ? 0 : first[i];
        const f32x4 a = *reinterpret_cast<const f32x4*>(src + f0);
        const f32x4 b = *reinterpret_cast<const f32x4*>(src + f0 + 4);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          vals[i][j] += hole ? 0.f : a[j];
          vals[i][4 + j] += hole ? 0.f : b[j];
        }
      }
    }
  }
  float mx = 0.f;
#pragma unroll
  for (int i = 0; i < kUnits; ++i) {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      vals[i][j] *= mscale;
      mx = fmaxf(mx, fabsf(vals[i][j]));
    }
    if (mat_out && !(kHoles && first[i] < 0)) {
      if (c_fast) {
#pragma unroll
        for (int j = 0; j < 8; ++j) mat_out[first[i] + j * rstep] = vals[i][j];
      } else {
        *reinterpret_cast<f32x4*>(mat_out + first[i]) = f32x4{vals[i][0], vals[i][1], vals[i][2], vals[i][3]};
        *reinterpret_cast<f32x4*>(mat_out + first[i] + 4) = f32x4{vals[i][4], vals[i][5], vals[i][6], vals[i][7]};
      }
    }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off));
  if (lane == 0) lds_max[wave] = mx;
  __syncthreads();
  mx = lds_max[0];
#pragma unroll
  for (int w = 1; w < NT / 64; ++w) mx = fmaxf(mx, lds_max[w]);
  float norm = 1.f;  // also when M is zero or not finite
  if (mx > 0.f && mx < 3.0e38f) {
    int e;
    frexpf(mx, &e);
    norm = ldexpf(1.f, 4 - e);
  }
#pragma unroll
  for (int i = 0; i < kUnits; ++i) {
    const int u = tid + NT * i;
    const int rg = c_fast ? u / DC : u % (DR / 8), cc = c_fast ? u % DC : u / (DR / 8);
    const int kbA = rg / (DR / 16), ks = rg % (DR / 16);
    const int kbC = cc / (DC / 2), rem = cc % (DC / 2);
    const int b = rem >> 4, m = 8 * ((rem & 15) >> 2) + 4 * kbC + (rem & 3);
    const int f = b * KS + ks, l = m + 32 * kbA;
    u32x4 whi, wlo;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float v0 = vals[i][2 * j] * norm, v1 = vals[i][2 * j + 1] * norm;
      const T h0 = (T)v0, h1 = (T)v1;
      whi[j] = pack2<T>((float)h0, (float)h1);
      wlo[j] = pack2<T>(v0 - (float)h0, v1 - (float)h1);
    }
    *reinterpret_cast<u32x4*>(lds_opnd + ((2 * f + 0) * 64 + l) * 16) = whi;
    *reinterpret_cast<u32x4*>(lds_opnd + ((2 * f + 1) * 64 + l) * 16) = wlo;
  }
  return 1.f / norm;
}

// km as 16-bit hi/lo pairs (for v_dot2) : pairs[0][e] = hi(km[2e], km[2e+1]), pairs[1][e] = lo
// `src` may be the vector part of the first of `nsum` partials (see build_operand);
// the sum times `vscale` is the vector.  It is stored as pairs (when `pairs`), as
// fp32 in LDS (when `f32`) and to memory (when `vec_out`).
// The LDS copies hold DP >= D entries (DP = 0 stands for D), zero past the first D, or
// (repeat) the D entries over and over.
template <typename T, int NT = kThreads>
__device__ __forceinline__ void build_vec(uint32_t* pairs, float* f32, const float* __restrict__ src,
                                          int D, int nsum = 1, int64_t sum_stride = 0,
                                          float vscale = 1.f, float* vec_out = nullptr, int DP = 0,
                                          bool repeat = false) {
  if (DP == 0) DP = D;
  for (int e = threadIdx.x; e < DP / 2; e += NT) {
    float a = 0.f, b = 0.f;
    const bool real = repeat || 2 * e < D;
    const int se = repeat ? (2 * e) % D : 2 * e;
    for (int c = 0; real && c < nsum; ++c) {
      a += src[(int64_t)c * sum_stride + se];
      b += src[(int64_t)c * sum_stride + se + 1];
    }
    a *= vscale;
    b *= vscale;
    if (pairs) {
      const T ah = (T)a, bh = (T)b;
      pairs[e] = pack2<T>((float)ah, (float)bh);
      pairs[DP / 2 + e] = pack2<T>(a - (float)ah, b - (float)bh);
    }
    if (f32) {
      f32[2 * e] = a;
      f32[2 * e + 1] = b;
    }
    if (vec_out && real && 2 * e < D) {
      vec_out[2 * e] = a;
      vec_out[2 * e + 1] = b;
    }
  }
}

// Denominator rows of the decoupled operator (DEN): with 64 x 64 tiles they are staged through LDS
// like the numerator rows; with a 128-wide side there is no LDS for a second tile per wave, and
// z_t = q_t . km is computed from the flat registers the rows were loaded into instead (the
// lanes that hold the 16-byte pieces of one row add their partial dot products; kDenFlat).
template <int DR, int DC, bool DEN> constexpr bool den_flat() { return DEN && !(DR == 64 && DC == 64); }
template <int DR, int DC, bool DEN, int WAVES, bool GATE = false> struct RowsLayout {
  static constexpr int KS = DR / 16, NB = DC / 32;
  static constexpr int kStage = 32 * 2 * (DR > DC ? DR : DC);  // one 32-token tile of the wider side
  static constexpr int kOpnd = NB * KS * 2 * 1024;
  static constexpr int kStages = kOpnd;
  static constexpr int kKm = kStages + WAVES * ((DEN && !den_flat<DR, DC, DEN>()) || GATE ? 2 : 1) * kStage;
  static constexpr int kAdd = kKm + DR * 4;
  static constexpr int kMax = kAdd + DC * 4;
  static constexpr int kZrow = kMax + 64;                                       // [WAVES][32] z of the wave's tile
  static constexpr int kLpt = kZrow + (den_flat<DR, DC, DEN>() ? WAVES * 128 : 0);
  static constexpr int kTotal = kLpt + (kLptMax + 1) * 4;
};

// One launch can carry two independent jobs of the same shape (the dk and dv
// products of backward pass B): workgroups [0, wgs_per_job) run job0, the rest job1.
// PAD = true: rows are dr (x) and dc (out) elements long in memory, multiples of 8 below the
// template's DR, DC; the staged tiles keep the padded width, with zeros in the padding.
// PAIR = true (dense tensors, 32 x 32 heads, DR = DC = 64): a 64-wide row of the kernel is two
// consecutive tokens of the head, the operand is blockdiag(M, M), and because a lane's z and
// its output features both belong to one half of the row, the halves never mix: the kernel
// streams full 128-byte rows at the cost of multiplying zeros.  `chunk` counts row pairs; an
// odd length leaves the second half of the last pair out.  No partial sums in the prologue.
// FMAP = true: the rows of x arrive before the feature map and are mapped (phi_pair) on their way into LDS.
template <typename T, int DR, int DC, bool NORM, bool DEN, int WAVES, bool PAD = false,
          int PF = (DR == 128 && DC == 128) ? FBLA_ROWS_PF128 : FBLA_ROWS_PF, bool PAIR = false, bool FMAP = false,
          bool GATE = false>
__global__ __launch_bounds__(WAVES * 64, (FBLA_ROWS_OCC4 && DR == 64 && DC == 64 && !DEN && !GATE) ? 4 : 1) void rows_kernel(Prob p, RowsJob job0, RowsJob job1,
                                                          int wgs_per_job, int chunk, int nchunks,
                                                          int dr_true, int dc_true) {
  static_assert(!PAIR || (DR == 64 && DC == 64 && !PAD), "pair mode: two 32-wide rows per 64-wide row");
  static_assert(!FMAP || (!DEN && !PAD && !PAIR), "feature map on load: plain rows only");
  static_assert(!GATE || (!DEN && !PAD && !PAIR && DR == DC), "gated output: plain square tiles only");

  const int dr = PAD ? dr_true : (PAIR ? 32 : DR), dc = PAD ? dc_true : (PAIR ? 32 : DC);
  const int dpk = PAD ? (p.DK <= 64 ? 64 : 128) : p.DK;  // padded length of the km / dkm vector
  using LY = RowsLayout<DR, DC, DEN, WAVES, GATE>;
  const bool second = (int)blockIdx.x >= wgs_per_job;
  const RowsJob& job = second ? job1 : job0;
  // FMAP and GATE together (pass B of a backward given the rows before the map): a job maps its x rows
  // when job.map_x is set, and its gate rows arrive before the map too
  const bool map_x = FMAP && (!GATE || job.map_x);
  const int wg = second ? blockIdx.x - wgs_per_job : blockIdx.x;
  constexpr int NT = WAVES * 64;
  constexpr int KS = DR / 16;  // k-steps
  constexpr int NB = DC / 32;  // output blocks
  constexpr int XROWB = DR * 2, OROWB = DC * 2;
  constexpr int XCH = XROWB / 16, OCH = OROWB / 16;  // 16-byte chunks per row
  constexpr int kStage = LY::kStage;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  unsigned char* lds_opnd = smem;
  uint32_t* lds_km = reinterpret_cast<uint32_t*>(smem + LY::kKm);  // [2][DR/2]
  float* lds_add = reinterpret_cast<float*>(smem + LY::kAdd);
  float* lds_max = reinterpret_cast<float*>(smem + LY::kMax);

  const int wg_item = packed_item(p, wg, p.H * nchunks);
  const int wg_nh = wg_item / nchunks, c = wg_item - wg_nh * nchunks;
  const int h = wg_nh % p.H;
  const int n = lpt_sequence(p, wg_nh / p.H, reinterpret_cast<int*>(smem + LY::kLpt));
  const int nh = n * p.H + h;
  int64_t bos, row0, rstride;
  int len;
  seq_range(p, n, bos, len);
  const int nrows = PAIR ? (len + 1) >> 1 : len;  // rows of this kernel
  // interleaved walk: the nchunks workgroups of a head take every nchunks-th step of
  // 32 * WAVES rows (one moving window per head instead of nchunks distant streams)
  const bool il = (p.flags & kInterleave) != 0;
  const int t_begin = il ? c * (32 * WAVES) : c * chunk;
  const int t_stride = 32 * WAVES * (il ? nchunks : 1);
  if (t_begin >= nrows) {
    if (c == 0 && job.pnchunks > 0) {  // empty sequence: its state is zero
      if (job.mat_out)
        for (int e = threadIdx.x; e < dr * dc; e += NT) job.mat_out[(int64_t)nh * dr * dc + e] = 0.f;
      if (job.vec_out)
        for (int e = threadIdx.x; e < p.DK; e += NT) job.vec_out[(int64_t)nh * p.DK + e] = 0.f;
    }
    return;
  }
  const int t_end = il ? nrows : min(nrows, t_begin + chunk);
  row_base(p, n, h, bos, row0, rstride);
  // element offset of 16-byte piece `ch` of row `tok` (rows of `rowlen` elements), or -1 when
  // the piece does not exist
  auto piece = [&](int tok, int ch, int rowlen) -> int64_t {
    if constexpr (PAIR) {
      if (tok >= t_end || 2 * tok + (ch >> 2) >= len) return -1;
      return (row0 + 2 * (int64_t)tok) * 32 + ch * 8;
    } else {
      if (tok >= t_end || (PAD && ch * 8 >= rowlen)) return -1;
      return (row0 + (int64_t)tok * rstride) * rowlen + ch * 8;
    }
  };

  const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const bool has_add = job.addvec != nullptr || job.vec_is_add;  // the same for all lanes
  const T* x = (const T*)job.x;
  const T* xden = (const T*)job.xden;
  T* out = (T*)job.out;

  // 32-token sub-tiles, interleaved over the waves; the first one is requested
  // before the prologue so that its latency overlaps the operand build.
  const int ntok = lane & 31, kb = lane >> 5;  // MFMA view: token column, k half
  constexpr bool kDenFlat = den_flat<DR, DC, DEN>();
  unsigned char* stage = smem + LY::kStages + wave * ((DEN && !kDenFlat) || GATE ? 2 : 1) * kStage;
  unsigned char* stage_den = stage + kStage;
  float* zrow = reinterpret_cast<float*>(smem + LY::kZrow) + 32 * wave;  // kDenFlat only
  constexpr int XI = 32 * XCH / 64;  // flat 16-byte loads per lane per tile
  constexpr int OI = 32 * OCH / 64;

  auto load_tile = [&](u32x4(&dst)[XI], const T* src, int tok0) {
#pragma unroll
    for (int i = 0; i < XI; ++i) {
      const int q = lane + 64 * i, row = q / XCH, ch = q % XCH;
      const int64_t off = piece(tok0 + row, ch, dr);
      if (off >= 0) {
        dst[i] = load_stream<u32x4, kNtRowsLoad>(src + off);
      } else {
        dst[i] = u32x4{0u, 0u, 0u, 0u};
      }
    }
  };
  auto stash_tile = [&](const u32x4(&src)[XI], unsigned char* dstb) {
#pragma unroll
    for (int i = 0; i < XI; ++i) {
      const int q = lane + 64 * i, row = q / XCH, ch = q % XCH;
      *reinterpret_cast<u32x4*>(dstb + swz<XROWB>(row, ch)) = src[i];
    }
  };
  // Whole tiles of plain rows (every tile but a ragged last one): a wave-uniform tile address
  // plus one constant byte offset per lane, and a uniform step between the lane's pieces; no
  // bounds checks and no 64-bit address arithmetic in vector registers.
  const bool kFast = !PAD && !PAIR && rstride <= (1 << 15);  // lane offsets stay within 32 bits
  const uint32_t xrow_b = (uint32_t)rstride * (uint32_t)(XROWB), orow_b = (uint32_t)rstride * (uint32_t)(OROWB);
  const uint32_t xvoff = (uint32_t)(lane / XCH) * xrow_b + (uint32_t)(lane % XCH) * 16u;
  const uint32_t ovoff = DR == DC ? xvoff : (uint32_t)(lane / OCH) * orow_b + (uint32_t)(lane % OCH) * 16u;
  const uint32_t xstep = (uint32_t)(64 / XCH) * xrow_b, ostep = (uint32_t)(64 / OCH) * orow_b;
  auto tile_ptr = [&](const void* base, int tok0, int rowlen) -> const char* {
    return reinterpret_cast<const char*>(base) + ((row0 + (int64_t)tok0 * rstride) * rowlen) * (int64_t)sizeof(T);
  };
  auto load_tile_full = [&](u32x4(&dst)[XI], const T* src, int tok0) {
    const char* tp = tile_ptr(src, tok0, DR);
#pragma unroll
    for (int i = 0; i < XI; ++i) dst[i] = load_stream<u32x4, kNtRowsLoad>(tp + (size_t)(xvoff + (uint32_t)i * xstep));
  };

  // PF register sets hold the tiles in flight: a tile is requested PF tiles ahead of its use
  int t0 = t_begin + 32 * wave;
  u32x4 xr[PF][XI], xd[DEN ? PF : 1][XI];
  // GATE: the mapped rows that scale this job's output (same pieces as the output's), or none
  const T* gate = GATE ? (const T*)job.gate : nullptr;
  u32x4 xg[GATE ? PF : 1][XI];
#pragma unroll
  for (int f = 0; f < PF; ++f)
    if (t0 + t_stride * f < t_end) {
      load_tile(xr[f], x, t0 + t_stride * f);
      if constexpr (DEN) load_tile(xd[f], xden, t0 + t_stride * f);
      if constexpr (GATE)
        if (gate) load_tile(xg[f], gate, t0 + t_stride * f);
    }

  // ---- prologue: matrix operand fragments, km pairs, addvec ----
  // Either the finished matrix / vectors are given, or the per-chunk partials of
  // the preceding reduction kernel, which are summed here in chunk order (every
  // workgroup of a head computes the same sums; chunk 0 also stores them).
  float denorm;
  if (job.pnchunks > 0) {
    const int E = dr * dc;
    const int64_t pstride = E + p.DK;
    const int nsum = min(job.pnchunks, (len + job.pchunk - 1) / job.pchunk);
    const float* part = job.mat + partial_slot(p, n, h, 0, job.pnchunks) * pstride;
    const int64_t sstride = pstride * partial_step(p);  // between the partials of consecutive chunks
    const bool writer = c == 0;
    denorm = build_operand<T, DR, DC, NT, PAD>(lds_opnd, lds_max, part, job.ld_r, job.ld_c, nsum, sstride,
                                               seq_scale(p, len),
                                               writer && job.mat_out ? job.mat_out + (int64_t)nh * E : nullptr,
                                               dr, dc);
    const float inv_len = 1.0f / (float)len;
    float* vout = writer && job.vec_out ? job.vec_out + (int64_t)nh * p.DK : nullptr;
    if (NORM || job.vec_is_add || vout)
      build_vec<T, NT>(NORM ? lds_km : nullptr, job.vec_is_add ? lds_add : nullptr, part + E, p.DK,
                       nsum, sstride, inv_len, vout, dpk);
    if (!job.vec_is_add)
      for (int e = tid; e < DC; e += NT) lds_add[e] = 0.f;
  } else {
    denorm = build_operand<T, DR, DC, NT, PAD, PAIR>(lds_opnd, lds_max, job.mat + (int64_t)nh * dr * dc,
                                                     job.ld_r, job.ld_c, 1, 0, 1.f, nullptr, dr, dc);
    if constexpr (NORM)
      build_vec<T, NT>(lds_km, nullptr, job.km + (int64_t)nh * dr, dr, 1, 0, 1.f, nullptr, DR, PAIR);
    for (int e = tid; e < DC; e += NT)
      lds_add[e] = (job.addvec && (PAIR || e < dc))
                       ? job.addvec[(int64_t)nh * dc + (PAIR ? e % 32 : e)] * job.add_scale
                       : 0.f;
  }
  __syncthreads();

  // ---- main loop ----
  // one tile: its rows move from the register set to the staging area, the set is refilled
  // with the tile PF steps ahead, then the tile is multiplied and stored
  auto tile_step = [&](u32x4(&xcur)[XI], u32x4(&dcur)[XI], u32x4(&gcur)[XI]) {
    wave_sync();  // previous tile's staging reads are done
    if constexpr (FMAP) {  // (rows past the end become phi(0) = 1: their outputs are not stored)
      if (map_x) {  // the same for all lanes
#pragma unroll
        for (int i = 0; i < XI; ++i)
#pragma unroll
          for (int w = 0; w < 4; ++w) xcur[i][w] = phi_pair<T>(xcur[i][w]);
      }
    }
    stash_tile(xcur, stage);
    if constexpr (DEN && !kDenFlat) stash_tile(dcur, stage_den);
    if constexpr (GATE) {
      if (gate) stash_tile(gcur, stage_den);  // (the same for all lanes) to be read per token below
    }
    if constexpr (kDenFlat) {
      // piece i of this lane is chunk lane % XCH of row lane / XCH + (64 / XCH) i: its dot product
      // with the km values of that chunk, then the sum over the XCH lanes of the row
      const u32x4 khf = *reinterpret_cast<const u32x4*>(&lds_km[4 * (lane % XCH)]);
      const u32x4 klf = *reinterpret_cast<const u32x4*>(&lds_km[DR / 2 + 4 * (lane % XCH)]);
#pragma unroll
      for (int i = 0; i < XI; ++i) {
        float a = 0.f;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
          a = Ops<T>::dot2(dcur[i][w], khf[w], a);
          a = Ops<T>::dot2(dcur[i][w], klf[w], a);
        }
#pragma unroll
        for (int off = XCH / 2; off > 0; off >>= 1) a += __shfl_xor(a, off);
        if (lane % XCH == 0) zrow[lane / XCH + (64 / XCH) * i] = a;
      }
    }
    const int tn = t0 + t_stride * PF;
    if ((FBLA_ROWS_FAST & 1) && !NORM && kFast && tn + 32 <= t_end) {
      load_tile_full(xcur, x, tn);
      if constexpr (DEN) load_tile_full(dcur, xden, tn);
    } else if (tn < t_end) {
      load_tile(xcur, x, tn);
      if constexpr (DEN) load_tile(dcur, xden, tn);
    }
    if constexpr (GATE) {
      if (gate && tn < t_end) load_tile(gcur, gate, tn);
    }
    wave_sync();

    f32x16 acc[NB];
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[b][r] = 0.f;
    float z = 0.f;
    // the LDS reads of k-step s+1 are issued before the MFMAs of step s, so that their latency
    // runs under the multiplications (two register sets, static indices after unrolling)
    struct Step {
      u32x4 bq, bd, kh, kl, ah[NB], al[NB];
    } st[2];
    auto fetch_step = [&](int s, Step& f) {
      f.bq = *reinterpret_cast<const u32x4*>(stage + swz<XROWB>(ntok, KS * kb + s));
#pragma unroll
      for (int b = 0; b < NB; ++b) {
        f.ah[b] = *reinterpret_cast<const u32x4*>(lds_opnd + ((2 * (b * KS + s) + 0) * 64 + lane) * 16);
        f.al[b] = *reinterpret_cast<const u32x4*>(lds_opnd + ((2 * (b * KS + s) + 1) * 64 + lane) * 16);
      }
      if constexpr (NORM && !kDenFlat) {
        if constexpr (DEN) f.bd = *reinterpret_cast<const u32x4*>(stage_den + swz<XROWB>(ntok, KS * kb + s));
        f.kh = *reinterpret_cast<const u32x4*>(&lds_km[(DR / 4) * kb + 4 * s]);
        f.kl = *reinterpret_cast<const u32x4*>(&lds_km[DR / 2 + (DR / 4) * kb + 4 * s]);
      }
    };
    fetch_step(0, st[0]);
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      if (s + 1 < KS) fetch_step(s + 1, st[(s + 1) & 1]);
      __builtin_amdgcn_sched_barrier(0);  // keep the reads above ahead of the MFMAs below
      const Step& f = st[s & 1];
      const u32x4 bq = f.bq;
#pragma unroll
      for (int b = 0; b < NB; ++b) {
        acc[b] = Ops<T>::mma(f.ah[b], bq, acc[b]);
        acc[b] = Ops<T>::mma(f.al[b], bq, acc[b]);
      }
      if constexpr (NORM && !kDenFlat) {
        u32x4 bd = bq;
        if constexpr (DEN) bd = f.bd;
        const u32x4 kh = f.kh, kl = f.kl;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          z = Ops<T>::dot2(bd[i], kh[i], z);
          z = Ops<T>::dot2(bd[i], kl[i], z);
        }
      }
    }
    float rs = denorm;
    if constexpr (NORM) {
      if constexpr (kDenFlat) z = zrow[ntok];  // written before the wave_sync above
      else if constexpr (!PAIR) z = sum_halves(z);  // pair mode: each half row has its own z
      rs = denorm / (z + p.eps);
    }
    wave_sync();  // all lanes have read their x chunks; staging is reused for out
    if (GATE && gate) {  // out = (acc * rs + add) * phi'(x): everything before the one rounding
      // phi'(x) = 1 for x > 0, exp(x) otherwise: from x itself (FMAP), or as min(phi(x), 1) from the mapped value
      auto dphi = [](float g) { return FMAP ? (g > 0.f ? 1.f : __expf(g)) : fminf(g, 1.f); };
#pragma unroll
      for (int b = 0; b < NB; ++b) {
        u32x4 w0, w1;
        const float* av = &lds_add[(DC / 2) * kb + 16 * b];
        const u32x4 g0 = *reinterpret_cast<const u32x4*>(stage_den + swz<OROWB>(ntok, (OCH / 2) * kb + 2 * b));
        const u32x4 g1 = *reinterpret_cast<const u32x4*>(stage_den + swz<OROWB>(ntok, (OCH / 2) * kb + 2 * b + 1));
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          w0[i] = pack2<T>(fmaf(acc[b][2 * i], rs, av[2 * i]) * dphi(Ops<T>::lo(g0[i])),
                           fmaf(acc[b][2 * i + 1], rs, av[2 * i + 1]) * dphi(Ops<T>::hi(g0[i])));
          w1[i] = pack2<T>(fmaf(acc[b][8 + 2 * i], rs, av[8 + 2 * i]) * dphi(Ops<T>::lo(g1[i])),
                           fmaf(acc[b][8 + 2 * i + 1], rs, av[8 + 2 * i + 1]) * dphi(Ops<T>::hi(g1[i])));
        }
        *reinterpret_cast<u32x4*>(stage + swz<OROWB>(ntok, (OCH / 2) * kb + 2 * b)) = w0;
        *reinterpret_cast<u32x4*>(stage + swz<OROWB>(ntok, (OCH / 2) * kb + 2 * b + 1)) = w1;
      }
    } else if (has_add) {  // only the dk job of the backward adds a row (dkm / L)
#pragma unroll
      for (int b = 0; b < NB; ++b) {
        u32x4 w0, w1;
        const float* av = &lds_add[(DC / 2) * kb + 16 * b];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          w0[i] = pack2<T>(fmaf(acc[b][2 * i], rs, av[2 * i]), fmaf(acc[b][2 * i + 1], rs, av[2 * i + 1]));
          w1[i] = pack2<T>(fmaf(acc[b][8 + 2 * i], rs, av[8 + 2 * i]),
                           fmaf(acc[b][8 + 2 * i + 1], rs, av[8 + 2 * i + 1]));
        }
        *reinterpret_cast<u32x4*>(stage + swz<OROWB>(ntok, (OCH / 2) * kb + 2 * b)) = w0;
        *reinterpret_cast<u32x4*>(stage + swz<OROWB>(ntok, (OCH / 2) * kb + 2 * b + 1)) = w1;
      }
    } else {
#pragma unroll
      for (int b = 0; b < NB; ++b) {
        u32x4 w0, w1;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          w0[i] = pack2<T>(acc[b][2 * i] * rs, acc[b][2 * i + 1] * rs);
          w1[i] = pack2<T>(acc[b][8 + 2 * i] * rs, acc[b][8 + 2 * i + 1] * rs);
        }
        *reinterpret_cast<u32x4*>(stage + swz<OROWB>(ntok, (OCH / 2) * kb + 2 * b)) = w0;
        *reinterpret_cast<u32x4*>(stage + swz<OROWB>(ntok, (OCH / 2) * kb + 2 * b + 1)) = w1;
      }
    }
    wave_sync();
    u32x4 wout[OI];  // all LDS reads first (one wait), then the stores
#pragma unroll
    for (int i = 0; i < OI; ++i) {
      const int q = lane + 64 * i;
      wout[i] = *reinterpret_cast<const u32x4*>(stage + swz<OROWB>(q / OCH, q % OCH));
    }
    if ((FBLA_ROWS_FAST & 2) && !NORM && kFast && t0 + 32 <= t_end) {
      char* tp = const_cast<char*>(tile_ptr(out, t0, DC));
#pragma unroll
      for (int i = 0; i < OI; ++i) store_row16<kNtRowsStore>(tp + (size_t)(ovoff + (uint32_t)i * ostep), wout[i]);
    } else {
#pragma unroll
      for (int i = 0; i < OI; ++i) {
        const int q = lane + 64 * i, row = q / OCH, ch = q % OCH;
        const int64_t off = piece(t0 + row, ch, dc);
        if (off >= 0) store_row16<kNtRowsStore>(out + off, wout[i]);
      }
    }
    t0 += t_stride;
  };
  while (t0 < t_end) {
#pragma unroll
    for (int f = 0; f < PF; ++f)
      if (t0 < t_end) tile_step(xr[f], xd[DEN ? f : 0], xg[GATE ? f : 0]);
  }
}

// ===========================================================================
// rows kernel for 128 x 128 matrices (not the decoupled operator's separate denominator rows)
// ===========================================================================
// The general kernel keeps the 64 KiB operand in LDS and lets every wave multiply its own tile
// by all of it (64 operand reads per tile, one eight-wave workgroup per CU).  Here a workgroup of
// four waves shares steps of 64 rows and two workgroups share a CU: the operand is built in LDS
// once, wave w keeps the fragments of output block w (32 of the 128 output columns) in 64
// registers, and the LDS becomes the row tiles.  Per step: the rows arrive flat and are staged
// (z_t = x_t . km is added up from the flat pieces on the way), every wave multiplies both
// tiles by its block, scales, adds, packs its 32 columns of every row into a staging step, and
// whole rows leave from there.  Two barriers per step; the x steps alternate between two buffers.
struct Rows128Layout {
  static constexpr int kOpnd = 4 * 8 * 2 * 1024;  // 4 blocks x 8 k-steps x (hi, lo) fragments
  static constexpr int kTile = 32 * 256;
  static constexpr int kStep = 2 * kTile;
  static constexpr int kX = 0;                  // x steps [2]
  static constexpr int kOut = 2 * kStep;        // output staging
  static constexpr int kKm = kOpnd;             // km as 16-bit pairs [2][64]
  static constexpr int kAdd = kKm + 128 * 4;    // row added to every output row [128]
  static constexpr int kZ = kAdd + 128 * 4;     // z of the step's rows [2][64]
  static constexpr int kMax = kZ + 2 * 64 * 4;
  static constexpr int kLpt = kMax + 64;
  static constexpr int kTotal = kLpt + (kLptMax + 1) * 4;
  static_assert(kOut + kStep <= kOpnd, "tiles live where the operand was built");
  static_assert(2 * kTotal <= 160 * 1024, "two workgroups per CU");
};

template <typename T, bool NORM, bool PAD>
__global__ __launch_bounds__(kThreads, 2) void rows128_kernel(Prob p, RowsJob job0, RowsJob job1, int wgs_per_job,
                                                              int chunk, int nchunks, int dr_true, int dc_true) {
  using LY = Rows128Layout;
  constexpr int KS = 8, ROWB = 256, NT = kThreads;
  const int dr = PAD ? dr_true : 128, dc = PAD ? dc_true : 128;
  const int dpk = PAD ? (p.DK <= 64 ? 64 : 128) : p.DK;  // padded length of the km / dkm vector
  const bool second = (int)blockIdx.x >= wgs_per_job;
  const RowsJob& job = second ? job1 : job0;
  const int wg = second ? blockIdx.x - wgs_per_job : blockIdx.x;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  uint32_t* lds_km = reinterpret_cast<uint32_t*>(smem + LY::kKm);
  float* lds_add = reinterpret_cast<float*>(smem + LY::kAdd);
  float* lds_z = reinterpret_cast<float*>(smem + LY::kZ);
  float* lds_max = reinterpret_cast<float*>(smem + LY::kMax);

  const int wg_item = packed_item(p, wg, p.H * nchunks);
  const int wg_nh = wg_item / nchunks, c = wg_item - wg_nh * nchunks;
  const int h = wg_nh % p.H;
  const int n = lpt_sequence(p, wg_nh / p.H, reinterpret_cast<int*>(smem + LY::kLpt));
  const int nh = n * p.H + h;
  int64_t bos, row0, rstride;
  int len;
  seq_range(p, n, bos, len);
  const int t_begin = c * chunk;
  if (t_begin >= len) {
    if (c == 0 && job.pnchunks > 0) {  // empty sequence: its state is zero
      if (job.mat_out)
        for (int e = threadIdx.x; e < dr * dc; e += NT) job.mat_out[(int64_t)nh * dr * dc + e] = 0.f;
      if (job.vec_out)
        for (int e = threadIdx.x; e < p.DK; e += NT) job.vec_out[(int64_t)nh * p.DK + e] = 0.f;
    }
    return;
  }
  const int t_end = min(len, t_begin + chunk);
  row_base(p, n, h, bos, row0, rstride);

  const int tid = threadIdx.x, blk = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int ntok = lane & 31, kb = lane >> 5;
  const bool has_add = job.addvec != nullptr || job.vec_is_add;  // the same for all lanes
  const T* x = (const T*)job.x;
  T* out = (T*)job.out;

  // The workgroup moves the 1024 16-byte pieces of a step's 64 rows: thread t takes pieces
  // t + 256 i, i.e. chunk t % 16 of rows t / 16 + 16 i: the step's uniform address plus a uniform
  // i-th distance plus the lane's one constant byte offset (32 bits: the host keeps packed
  // tensors with more than 65536 heads away from this kernel).
  const int prow = tid >> 4, pch = tid & 15;
  const uint32_t xrow_b = (uint32_t)rstride * (uint32_t)dr * 2u, orow_b = (uint32_t)rstride * (uint32_t)dc * 2u;
  const uint32_t xvoff = (uint32_t)prow * xrow_b + (uint32_t)pch * 16u;
  const uint32_t ovoff = PAD ? (uint32_t)prow * orow_b + (uint32_t)pch * 16u : xvoff;
  const bool x_piece = !PAD || pch * 8 < dr, o_piece = !PAD || pch * 8 < dc;
  auto step_ptr = [&](const void* base, int tok0, int rowlen) -> const char* {
    return reinterpret_cast<const char*>(base) + ((row0 + (int64_t)tok0 * rstride) * rowlen) * (int64_t)sizeof(T);
  };
  auto load_step = [&](u32x4(&dst)[4], int tok0) {
    const char* tp = step_ptr(x, tok0, dr);
    const int rows = t_end - tok0;  // rows of this step that exist (may be <= 0)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      dst[i] = u32x4{0u, 0u, 0u, 0u};
      if (x_piece && prow + 16 * i < rows) dst[i] = load_stream<u32x4, kNtRowsLoad>(tp + (size_t)(16 * i) * xrow_b + xvoff);
    }
  };

  u32x4 rx[4];
  load_step(rx, t_begin);

  // ---- prologue: matrix operand fragments, km pairs, addvec (as in rows_kernel) ----
  float denorm;
  if (job.pnchunks > 0) {
    const int E = dr * dc;
    const int64_t pstride = E + p.DK;
    const int nsum = min(job.pnchunks, (len + job.pchunk - 1) / job.pchunk);
    const float* part = job.mat + partial_slot(p, n, h, 0, job.pnchunks) * pstride;
    const int64_t sstride = pstride * partial_step(p);  // between the partials of consecutive chunks
    const bool writer = c == 0;
    denorm = build_operand<T, 128, 128, NT, PAD>(smem, lds_max, part, job.ld_r, job.ld_c, nsum, sstride,
                                                 seq_scale(p, len),
                                                 writer && job.mat_out ? job.mat_out + (int64_t)nh * E : nullptr, dr,
                                                 dc);
    const float inv_len = 1.0f / (float)len;
    float* vout = writer && job.vec_out ? job.vec_out + (int64_t)nh * p.DK : nullptr;
    if (NORM || job.vec_is_add || vout)
      build_vec<T, NT>(NORM ? lds_km : nullptr, job.vec_is_add ? lds_add : nullptr, part + E, p.DK, nsum, sstride,
                       inv_len, vout, dpk);
    if (!job.vec_is_add)
      for (int e = tid; e < 128; e += NT) lds_add[e] = 0.f;
  } else {
    denorm = build_operand<T, 128, 128, NT, PAD>(smem, lds_max, job.mat + (int64_t)nh * dr * dc, job.ld_r, job.ld_c,
                                                 1, 0, 1.f, nullptr, dr, dc);
    if constexpr (NORM) build_vec<T, NT>(lds_km, nullptr, job.km + (int64_t)nh * dr, dr, 1, 0, 1.f, nullptr, 128);
    for (int e = tid; e < 128; e += NT)
      lds_add[e] = (job.addvec && e < dc) ? job.addvec[(int64_t)nh * dc + e] * job.add_scale : 0.f;
  }
  __syncthreads();
  u32x4 sh[KS], sl[KS];  // output block blk: columns 64 kb' + 16 blk + 0..15 of lane (row, kb')
#pragma unroll
  for (int s = 0; s < KS; ++s) {
    const int f = blk * KS + s;
    sh[s] = *reinterpret_cast<const u32x4*>(smem + ((2 * f + 0) * 64 + lane) * 16);
    sl[s] = *reinterpret_cast<const u32x4*>(smem + ((2 * f + 1) * 64 + lane) * 16);
  }
  // the row added to this lane's 16 columns, and the km pairs of this thread's chunk of a row
  float addv[16];
#pragma unroll
  for (int r = 0; r < 16; ++r) addv[r] = lds_add[64 * kb + 16 * blk + r];
  u32x4 kmh = u32x4{0u, 0u, 0u, 0u}, kml = kmh;
  if constexpr (NORM) {
    kmh = *reinterpret_cast<const u32x4*>(&lds_km[4 * pch]);
    kml = *reinterpret_cast<const u32x4*>(&lds_km[64 + 4 * pch]);
  }
  __syncthreads();  // the operand has left LDS

  unsigned char* ostage = smem + LY::kOut;
  int buf = 0;
  for (int base = t_begin; base < t_end; base += 64) {
    unsigned char* xt = smem + LY::kX + buf * LY::kStep;
    float* zrow = lds_z + 64 * buf;
#pragma unroll
    for (int i = 0; i < 4; ++i) *reinterpret_cast<u32x4*>(xt + swz<ROWB>(prow + 16 * i, pch)) = rx[i];
    if constexpr (NORM) {
      // piece i of this thread is chunk pch of row prow + 16 i: its dot product with the km values
      // of that chunk, then the sum over the 16 lanes of the row
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float a = 0.f;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
          a = Ops<T>::dot2(rx[i][w], kmh[w], a);
          a = Ops<T>::dot2(rx[i][w], kml[w], a);
        }
#pragma unroll
        for (int off = 8; off > 0; off >>= 1) a += __shfl_xor(a, off);
        if (pch == 0) zrow[prow + 16 * i] = a;
      }
    }
    load_step(rx, base + 64);
    __syncthreads();  // the step and its z are in LDS; the staging step has been read out

    // this lane gets columns 64 kb + 16 blk + 0..15 of row ntok of both tiles
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      f32x16 acc;
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[r] = 0.f;
#pragma unroll
      for (int s = 0; s < KS; ++s) {
        const u32x4 bq = *reinterpret_cast<const u32x4*>(xt + t * LY::kTile + swz<ROWB>(ntok, KS * kb + s));
        acc = Ops<T>::mma(sh[s], bq, acc);
        acc = Ops<T>::mma(sl[s], bq, acc);
      }
      float rs = denorm;
      if constexpr (NORM) rs = denorm / (zrow[32 * t + ntok] + p.eps);
#pragma unroll
      for (int ch = 0; ch < 2; ++ch) {
        u32x4 w;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int c0 = 8 * ch + 2 * i;
          float v0 = acc[c0] * rs, v1 = acc[c0 + 1] * rs;
          if (has_add) {
            v0 += addv[c0];
            v1 += addv[c0 + 1];
          }
          w[i] = pack2<T>(v0, v1);
        }
        *reinterpret_cast<u32x4*>(ostage + t * LY::kTile + swz<ROWB>(ntok, 8 * kb + 2 * blk + ch)) = w;
      }
    }
    __syncthreads();  // the output rows are complete
    {
      char* tp = const_cast<char*>(step_ptr(out, base, dc));
      const int rows = t_end - base;
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (o_piece && prow + 16 * i < rows)
          store_row16<kNtRowsStore>(tp + (size_t)(16 * i) * orow_b + ovoff,
                                    *reinterpret_cast<const u32x4*>(ostage + swz<ROWB>(prow + 16 * i, pch)));
    }
    buf ^= 1;
  }
}

// ===========================================================================
// backward pass A
// ===========================================================================
// Per 32-token sub-tile (one wave):
//   token view (lane = token n, half kb):  g_t = dO_t S^T by MFMA, then in registers
//     P_t = q~_t . g_t,  z_t = q_t . km + eps,  dz_t = -P_t / z_t^2,
//     dq~_t = g_t / z_t (+ dz_t km),  and dO_t / z_t is written back to LDS as hi + lo;
//   feature view (lane = feature pair, registers = tokens): dS += q~^T (dO / z) by MFMA
//     with the same in-register transposition as the state kernel, dkm += dz_t q_t.
// dS and dkm partials leave through the same reduction as the forward state.
template <int C>
__device__ __forceinline__ void lds_rows(RowWords<C>& dst, const unsigned char* tile, int tok0,
                                         int pp) {
  constexpr int ROWB = C * 64;  // bytes per row: 32 lanes x C features x 2 bytes
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const int row = tok0 + j;
    if constexpr (C == 2) {
      dst.w[j][0] = *reinterpret_cast<const uint32_t*>(tile + swz<ROWB>(row, pp >> 2) + ((pp & 3) << 2));
    } else {
      const u32x2 x = *reinterpret_cast<const u32x2*>(tile + swz<ROWB>(row, pp >> 1) + ((pp & 1) << 3));
      dst.w[j][0] = x[0];
      dst.w[j][1] = x[1];
    }
  }
}

template <int DK, int DV, bool NORM, bool DEN, bool FUSED, bool LO = true> struct BwdALayout {
  static constexpr int KS = DV / 16, NB = DK / 32;
  static constexpr int kOpnd = NB * KS * 2 * 1024;
  static constexpr int kQ = 32 * DK * 2, kG = 32 * DV * 2;
  // (DEN without FUSED: the denominator rows stay in the flat registers they were loaded into)
  static constexpr int kWave = kQ + kG + (NORM && FUSED && LO ? kG : 0) + (DEN && FUSED ? kQ : 0) + 256;  // + dz[64]
  static constexpr int kKmPairs = kOpnd + kWaves * kWave;
  static constexpr int kKmF = kKmPairs + DK * 4;
  static constexpr int kMax = kKmF + DK * 4;
  static constexpr int kLpt = kMax + 64;
  static constexpr int kTotal = kLpt + (kLptMax + 1) * 4;
};

// FUSED = false runs the token view only (head dims whose dS accumulators do not
// fit one wave): it writes 1/z_t and dz_t per (token, head) row to `tokscal`
// ([2][total rows]) for scaled_state_kernel, and no partials.
// PAD = true: head dims p.DK, p.DV (multiples of 8) below the template's DK, DV, as in the
// other kernels: true row lengths in memory, zero padding in the staged tiles and operands.
// PAIR = true (dense tensors, 32 x 32 heads, DK = DV = 64, FUSED): two consecutive tokens per
// 64-wide row as in the rows kernel; the token view never mixes the halves of a row, the
// feature view accumulates blockdiag-shaped sums whose two diagonal 32 x 32 blocks are added
// before the store.  `chunk` counts row pairs.
// GATE = true: q are the mapped rows phi(x) and dq is wanted with respect to x: times min(q, 1).
// FMAP = true (with GATE): q are the rows x themselves and are mapped on their way into LDS.
template <typename T, int DK, int DV, bool NORM, bool DEN, bool FUSED, bool LO = true, bool PAD = false,
          bool PAIR = false, bool GATE = false, bool FMAP = false>
__global__ __launch_bounds__(kThreads, (FBLA_BWDA_OCC3 && FUSED && !DEN && !LO) ? 3 : 2) void bwd_a_kernel(
    Prob p, const T* __restrict__ qn, const T* __restrict__ qd, const T* __restrict__ dout,
    const float* __restrict__ S, const float* __restrict__ km, T* __restrict__ dqn,
    T* __restrict__ dqd, float* __restrict__ partial, float* __restrict__ tokscal,
    int64_t total_rows, float* fin_mat, float* fin_vec, int chunk, int nchunks) {
  using LY = BwdALayout<DK, DV, NORM, DEN, FUSED, LO>;
  constexpr int KS = LY::KS, NB = LY::NB;
  constexpr int CK = DK / 32, CV = DV / 32;
  static_assert(!FUSED || (DK == 64 && DV == 64), "the fused form exists for 64 x 64 tiles (128 x 128: bwd_a128_kernel)");
  static_assert(!PAIR || (DK == 64 && DV == 64 && FUSED && !PAD), "pair mode: two 32-wide rows per 64-wide row");
  const int dk = PAD ? p.DK : (PAIR ? 32 : DK), dv = PAD ? p.DV : (PAIR ? 32 : DV);
  constexpr int QROWB = DK * 2, GROWB = DV * 2;
  constexpr int QCH = QROWB / 16, GCH = GROWB / 16;
  constexpr int QI = 32 * QCH / 64, GI = 32 * GCH / 64;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

  const int wg_item = packed_item(p, blockIdx.x, p.H * nchunks);
  const int wg_nh = wg_item / nchunks, c = wg_item - wg_nh * nchunks;
  const int h = wg_nh % p.H;
  const int n = lpt_sequence(p, wg_nh / p.H, reinterpret_cast<int*>(smem + LY::kLpt));
  const int nh = n * p.H + h;
  int64_t bos, row0, rstride;
  int len;
  seq_range(p, n, bos, len);
  const int nrows = PAIR ? (len + 1) >> 1 : len;  // rows of this kernel
  // interleaved walk: the nchunks workgroups of a head take every nchunks-th step of 128 rows
  const bool il = FUSED && (p.flags & kInterleave) != 0;
  const int t_begin = il ? c * (32 * kWaves) : c * chunk;
  const int t_stride = 32 * kWaves * (il ? nchunks : 1);
  if (t_begin >= nrows) {
    if (fin_mat && c == 0) {  // empty sequence: no gradient flows through its state
      for (int e = threadIdx.x; e < dk * dv; e += kThreads) fin_mat[(int64_t)nh * dk * dv + e] = 0.f;
      if (fin_vec)
        for (int e = threadIdx.x; e < dk; e += kThreads) fin_vec[(int64_t)nh * dk + e] = 0.f;
    }
    return;
  }
  const int t_end = il ? nrows : min(nrows, t_begin + chunk);
  row_base(p, n, h, bos, row0, rstride);
  // element offset of 16-byte piece `ch` of row `tok` (rows of `rowlen` elements), or -1 when
  // the piece does not exist
  auto piece = [&](int tok, int ch, int rowlen) -> int64_t {
    if constexpr (PAIR) {
      if (tok >= t_end || 2 * tok + (ch >> 2) >= len) return -1;
      return (row0 + 2 * (int64_t)tok) * 32 + ch * 8;
    } else {
      if (tok >= t_end || (PAD && ch * 8 >= rowlen)) return -1;
      return (row0 + (int64_t)tok * rstride) * rowlen + ch * 8;
    }
  };

  const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int ntok = lane & 31, kb = lane >> 5;

  unsigned char* lds_opnd = smem;
  unsigned char* qt = smem + LY::kOpnd + wave * LY::kWave;
  unsigned char* gt = qt + LY::kQ;             // dO, later dO/z (hi part)
  unsigned char* gl = gt + LY::kG;             // dO/z (lo part), NORM && FUSED only
  // Token view alone (not FUSED) with the decoupled operator: z_t = q_t . km comes from the flat
  // registers of the plain q rows (the lanes holding the pieces of a row add their partial dot
  // products) and dq = dz_t km is stored from the same flat layout: no LDS tile for plain q.
  constexpr bool kDenFlat = DEN && !FUSED;
  unsigned char* qdt = gl + (NORM && FUSED && LO ? LY::kG : 0);  // plain q, DEN && FUSED only
  float* dzs = reinterpret_cast<float*>(qdt + (DEN && FUSED ? LY::kQ : 0));  // [64]: dz (FUSED) or z | dz (kDenFlat)
  uint32_t* km_pairs = reinterpret_cast<uint32_t*>(smem + LY::kKmPairs);
  float* kmf = reinterpret_cast<float*>(smem + LY::kKmF);
  float* lds_max = reinterpret_cast<float*>(smem + LY::kMax);

  constexpr int AK = FUSED ? 2 : 1, AV = FUSED ? 2 : 1;  // one 64 x 64 block of dS per wave
  f32x16 acc[AK][AV];
#pragma unroll
  for (int a = 0; a < AK; ++a)
#pragma unroll
    for (int b = 0; b < AV; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.f;
  float dkm[2] = {0.f, 0.f};

  auto load_q = [&](u32x4(&dst)[QI], const T* src, int tok0) {
#pragma unroll
    for (int i = 0; i < QI; ++i) {
      const int q = lane + 64 * i, row = q / QCH, ch = q % QCH;
      const int64_t off = piece(tok0 + row, ch, dk);
      dst[i] = off >= 0 ? load_stream<u32x4, kNtPassALoad>(src + off) : u32x4{0u, 0u, 0u, 0u};
    }
  };
  auto load_g = [&](u32x4(&dst)[GI], const T* src, int tok0) {
#pragma unroll
    for (int i = 0; i < GI; ++i) {
      const int q = lane + 64 * i, row = q / GCH, ch = q % GCH;
      const int64_t off = piece(tok0 + row, ch, dv);
      dst[i] = off >= 0 ? load_stream<u32x4, kNtPassALoad>(src + off) : u32x4{0u, 0u, 0u, 0u};
    }
  };
  auto stash_q = [&](const u32x4(&src)[QI], unsigned char* dstb) {
#pragma unroll
    for (int i = 0; i < QI; ++i) {
      const int q = lane + 64 * i;
      *reinterpret_cast<u32x4*>(dstb + swz<QROWB>(q / QCH, q % QCH)) = src[i];
    }
  };
  auto stash_g = [&](const u32x4(&src)[GI], unsigned char* dstb) {
#pragma unroll
    for (int i = 0; i < GI; ++i) {
      const int q = lane + 64 * i;
      *reinterpret_cast<u32x4*>(dstb + swz<GROWB>(q / GCH, q % GCH)) = src[i];
    }
  };
  auto store_q = [&](const unsigned char* srcb, T* dst, int tok0) {
#pragma unroll
    for (int i = 0; i < QI; ++i) {
      const int q = lane + 64 * i, row = q / QCH, ch = q % QCH;
      const int64_t off = piece(tok0 + row, ch, dk);
      if (off >= 0)
        store_row16<kNtPassAStore>(dst + off, *reinterpret_cast<const u32x4*>(srcb + swz<QROWB>(row, ch)));
    }
  };
  // Whole tiles of plain rows: a wave-uniform tile address plus one constant byte offset per
  // lane and a uniform step between the lane's pieces (as in the rows kernel).
  const bool kFast = !PAD && !PAIR && rstride <= (1 << 15);  // lane offsets stay within 32 bits
  const uint32_t qrow_b = (uint32_t)rstride * (uint32_t)QROWB, grow_b = (uint32_t)rstride * (uint32_t)GROWB;
  const uint32_t qvoff = (uint32_t)(lane / QCH) * qrow_b + (uint32_t)(lane % QCH) * 16u;
  const uint32_t gvoff = (uint32_t)(lane / GCH) * grow_b + (uint32_t)(lane % GCH) * 16u;
  const uint32_t qstep = (uint32_t)(64 / QCH) * qrow_b, gstep = (uint32_t)(64 / GCH) * grow_b;
  auto tile_ptr = [&](const void* base, int tok0, int rowlen) -> const char* {
    return reinterpret_cast<const char*>(base) + ((row0 + (int64_t)tok0 * rstride) * rowlen) * (int64_t)sizeof(T);
  };
  auto load_q_full = [&](u32x4(&dst)[QI], const T* src, int tok0) {
    const char* tp = tile_ptr(src, tok0, DK);
#pragma unroll
    for (int i = 0; i < QI; ++i) dst[i] = load_stream<u32x4, kNtPassALoad>(tp + (size_t)(qvoff + (uint32_t)i * qstep));
  };
  auto load_g_full = [&](u32x4(&dst)[GI], const T* src, int tok0) {
    const char* tp = tile_ptr(src, tok0, DV);
#pragma unroll
    for (int i = 0; i < GI; ++i) dst[i] = load_stream<u32x4, kNtPassALoad>(tp + (size_t)(gvoff + (uint32_t)i * gstep));
  };
  auto store_q_full = [&](const unsigned char* srcb, T* dst, int tok0) {
    char* tp = const_cast<char*>(tile_ptr(dst, tok0, DK));
#pragma unroll
    for (int i = 0; i < QI; ++i) {
      const int q = lane + 64 * i;
      store_row16<kNtPassAStore>(tp + (size_t)(qvoff + (uint32_t)i * qstep),
                                 *reinterpret_cast<const u32x4*>(srcb + swz<QROWB>(q / QCH, q % QCH)));
    }
  };

  int t0 = t_begin + 32 * wave;
  u32x4 rq[QI], rg[GI], rd[QI];
  if (t0 < t_end) {
    load_q(rq, qn, t0);
    load_g(rg, dout, t0);
    if constexpr (DEN) load_q(rd, qd, t0);
  }

  // g_t = dO_t S^T: contraction over dv, M(r = dv, c = dk) = S[c][r]
  const float denorm = build_operand<T, DV, DK, kThreads, PAD, PAIR>(
      lds_opnd, lds_max, S + (int64_t)nh * dk * dv, 1, dv, 1, 0, 1.f, nullptr, dv, dk);
  if constexpr (NORM) {
    build_vec<T>(km_pairs, kmf, km + (int64_t)nh * dk, dk, 1, 0, 1.f, nullptr, DK, PAIR);
  }
  __syncthreads();

  static_assert(!FMAP || GATE, "q mapped on load: together with the gated dq");
  while (t0 < t_end) {
    wave_sync();  // the previous sub-tile's staged dq has been read out
    if constexpr (FMAP) {  // (rows past the end become phi(0) = 1: they are masked by rz = 0 and not stored)
#pragma unroll
      for (int i = 0; i < QI; ++i)
#pragma unroll
        for (int w = 0; w < 4; ++w) rq[i][w] = phi_pair<T>(rq[i][w]);
    }
    stash_q(rq, qt);
    stash_g(rg, gt);
    if constexpr (DEN && !kDenFlat) stash_q(rd, qdt);
    if constexpr (kDenFlat) {
      const u32x4 khf = *reinterpret_cast<const u32x4*>(&km_pairs[4 * (lane % QCH)]);
      const u32x4 klf = *reinterpret_cast<const u32x4*>(&km_pairs[DK / 2 + 4 * (lane % QCH)]);
#pragma unroll
      for (int i = 0; i < QI; ++i) {
        float a = 0.f;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
          a = Ops<T>::dot2(rd[i][w], khf[w], a);
          a = Ops<T>::dot2(rd[i][w], klf[w], a);
        }
#pragma unroll
        for (int off = QCH / 2; off > 0; off >>= 1) a += __shfl_xor(a, off);
        if (lane % QCH == 0) dzs[lane / QCH + (64 / QCH) * i] = a;
      }
    }
    const int tn = t0 + t_stride;
    auto request_next = [&]() {
      if (kFast && tn + 32 <= t_end) {
        load_q_full(rq, qn, tn);
        load_g_full(rg, dout, tn);
        if constexpr (DEN) load_q_full(rd, qd, tn);
      } else if (tn < t_end) {
        load_q(rq, qn, tn);
        load_g(rg, dout, tn);
        if constexpr (DEN) load_q(rd, qd, tn);
      }
    };
    if constexpr (FBLA_BWDA_NEXT_AT == 0) request_next();
    wave_sync();

    // ---- token view ----
    f32x16 g[NB];
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) g[b][r] = 0.f;
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      const u32x4 bq = *reinterpret_cast<const u32x4*>(gt + swz<GROWB>(ntok, KS * kb + s));
#pragma unroll
      for (int b = 0; b < NB; ++b) {
        const u32x4 ah = *reinterpret_cast<const u32x4*>(lds_opnd + ((2 * (b * KS + s) + 0) * 64 + lane) * 16);
        const u32x4 al = *reinterpret_cast<const u32x4*>(lds_opnd + ((2 * (b * KS + s) + 1) * 64 + lane) * 16);
        g[b] = Ops<T>::mma(ah, bq, g[b]);
        g[b] = Ops<T>::mma(al, bq, g[b]);
      }
    }
    if constexpr (FBLA_BWDA_NEXT_AT == 1) request_next();
    // this lane: g[token][c], c = (DK/2)*kb + 16b + r
    float rz = 1.f, dz = 0.f;
    if constexpr (NORM) {
      float P = 0.f, z = 0.f;
#pragma unroll
      for (int ch = 0; ch < QCH / 2; ++ch) {
        const u32x4 qw = *reinterpret_cast<const u32x4*>(qt + swz<QROWB>(ntok, (QCH / 2) * kb + ch));
        u32x4 qz = qw;
        if constexpr (DEN && !kDenFlat) qz = *reinterpret_cast<const u32x4*>(qdt + swz<QROWB>(ntok, (QCH / 2) * kb + ch));
        const u32x4 kh = *reinterpret_cast<const u32x4*>(&km_pairs[(DK / 4) * kb + 4 * ch]);
        const u32x4 kl = *reinterpret_cast<const u32x4*>(&km_pairs[DK / 2 + (DK / 4) * kb + 4 * ch]);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int c0 = 8 * ch + 2 * i;
          P = fmaf(Ops<T>::lo(qw[i]), g[c0 >> 4][c0 & 15], P);
          P = fmaf(Ops<T>::hi(qw[i]), g[c0 >> 4][(c0 & 15) + 1], P);
          if constexpr (!kDenFlat) {
            z = Ops<T>::dot2(qz[i], kh[i], z);
            z = Ops<T>::dot2(qz[i], kl[i], z);
          }
        }
      }
      if constexpr (!PAIR) {  // pair mode: each half row is a token of its own
        P = sum_halves(P);
        z = sum_halves(z);
      }
      if constexpr (kDenFlat) z = dzs[ntok];  // from the flat registers, before the wave_sync above
      if (PAIR ? (t0 + ntok < t_end && 2 * (t0 + ntok) + kb < len) : (t0 + ntok < t_end)) {
        rz = 1.f / (z + p.eps);
        dz = -(P * denorm) * rz * rz;
      } else {
        rz = 0.f;  // padding rows contribute nothing
      }
      if constexpr (FUSED) {
        if (PAIR || kb == 0) dzs[32 * (PAIR ? kb : 0) + ntok] = dz;
      } else {
        if (kb == 0 && t0 + ntok < t_end) {
          const int64_t row = row0 + (int64_t)(t0 + ntok) * rstride;
          tokscal[row] = rz;
          tokscal[total_rows + row] = dz;
        }
        if constexpr (kDenFlat) {
          if (kb == 0) dzs[32 + ntok] = dz;
        }
      }
    }
    // dq~ (and dq when decoupled), packed; staged after the feature view is done with qt
    uint32_t dqp[DK / 4], dqdp[DEN && !kDenFlat ? DK / 4 : 1];
    {
      const float gs = denorm * rz;
      static_assert(!GATE || (FUSED && !DEN && !PAD && !PAIR), "gated dq: the plain fused kernel only");
      u32x4 qmapped[GATE ? QCH / 2 : 1];  // this lane's half of its token's (mapped) q row, still in the tile
      if constexpr (GATE) {
#pragma unroll
        for (int ch = 0; ch < QCH / 2; ++ch)
          qmapped[ch] = *reinterpret_cast<const u32x4*>(qt + swz<QROWB>(ntok, (QCH / 2) * kb + ch));
      }
#pragma unroll
      for (int c2 = 0; c2 < DK / 4; ++c2) {
        const int c0 = 2 * c2;
        float v0 = g[c0 >> 4][c0 & 15] * gs, v1 = g[c0 >> 4][(c0 & 15) + 1] * gs;
        if constexpr (NORM) {
          const float d0 = dz * kmf[(DK / 2) * kb + c0], d1 = dz * kmf[(DK / 2) * kb + c0 + 1];
          if constexpr (DEN && !kDenFlat) {
            dqdp[c2] = pack2<T>(d0, d1);
          } else if constexpr (!DEN) {
            v0 += d0;
            v1 += d1;
          }
        }
        if constexpr (GATE) {  // phi'(x) = min(phi(x), 1)
          const uint32_t w = qmapped[c2 >> 2][c2 & 3];
          v0 *= fminf(Ops<T>::lo(w), 1.f);
          v1 *= fminf(Ops<T>::hi(w), 1.f);
        }
        dqp[c2] = pack2<T>(v0, v1);
      }
    }
    // dO / z as hi + lo, in place over this lane's own chunks of the dO tile
    if constexpr (NORM && FUSED) {
#pragma unroll
      for (int ch = 0; ch < GCH / 2; ++ch) {
        const int off = swz<GROWB>(ntok, (GCH / 2) * kb + ch);
        const u32x4 gw = *reinterpret_cast<const u32x4*>(gt + off);
        u32x4 wh, wl;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float a = Ops<T>::lo(gw[i]) * rz, b = Ops<T>::hi(gw[i]) * rz;
          const T ah = (T)a, bh = (T)b;
          wh[i] = pack2<T>((float)ah, (float)bh);
          wl[i] = pack2<T>(a - (float)ah, b - (float)bh);
        }
        *reinterpret_cast<u32x4*>(gt + off) = wh;
        if constexpr (LO) *reinterpret_cast<u32x4*>(gl + off) = wl;
      }
    }
    wave_sync();
    if constexpr (FBLA_BWDA_NEXT_AT == 2) request_next();

    // ---- feature view: two k-steps of 16 tokens ----
    if constexpr (FUSED) {
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      const int tok0 = 16 * ks + 8 * kb;
      RowWords<CK> qw;
      RowWords<CV> gh;
      lds_rows<CK>(qw, qt, tok0, ntok);
      lds_rows<CV>(gh, gt, tok0, ntok);
      u32x4 A[CK], Bh[CV];
      transpose_rows<CK>(qw, A);
      transpose_rows<CV>(gh, Bh);
#pragma unroll
      for (int a = 0; a < CK; ++a)
#pragma unroll
        for (int b = 0; b < CV; ++b) acc[a][b] = Ops<T>::mma(A[a], Bh[b], acc[a][b]);
      if constexpr (NORM) {
        if constexpr (LO) {
          RowWords<CV> glw;
          lds_rows<CV>(glw, gl, tok0, ntok);
          u32x4 Bl[CV];
          transpose_rows<CV>(glw, Bl);
#pragma unroll
          for (int a = 0; a < CK; ++a)
#pragma unroll
            for (int b = 0; b < CV; ++b) acc[a][b] = Ops<T>::mma(A[a], Bl[b], acc[a][b]);
        }
        if constexpr (DEN) lds_rows<CK>(qw, qdt, tok0, ntok);
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const float dzj = dzs[(PAIR ? 32 * (ntok >> 4) : 0) + tok0 + j];  // lanes 16.. hold the second halves
#pragma unroll
          for (int c2 = 0; c2 < CK / 2; ++c2) {
            dkm[2 * c2] = fmaf(dzj, Ops<T>::lo(qw.w[j][c2]), dkm[2 * c2]);
            dkm[2 * c2 + 1] = fmaf(dzj, Ops<T>::hi(qw.w[j][c2]), dkm[2 * c2 + 1]);
          }
        }
      }
    }
    }
    wave_sync();  // qt (and qdt) are free: stage dq through them
#pragma unroll
    for (int ch = 0; ch < QCH / 2; ++ch) {
      const int off = swz<QROWB>(ntok, (QCH / 2) * kb + ch);
      *reinterpret_cast<u32x4*>(qt + off) = u32x4{dqp[4 * ch], dqp[4 * ch + 1], dqp[4 * ch + 2], dqp[4 * ch + 3]};
      if constexpr (DEN && !kDenFlat)
        *reinterpret_cast<u32x4*>(qdt + off) =
            u32x4{dqdp[4 * ch], dqdp[4 * ch + 1], dqdp[4 * ch + 2], dqdp[4 * ch + 3]};
    }
    wave_sync();  // (also orders the dz values written to dzs[32..] before the reads below)
    if (kFast && t0 + 32 <= t_end) {
      store_q_full(qt, dqn, t0);
      if constexpr (DEN && !kDenFlat) store_q_full(qdt, dqd, t0);
    } else {
      store_q(qt, dqn, t0);
      if constexpr (DEN && !kDenFlat) store_q(qdt, dqd, t0);
    }
    if constexpr (kDenFlat) {
      // dq = dz_t km: piece i of this lane is chunk lane % QCH of row lane / QCH + (64 / QCH) i
      const float* kmc = kmf + 8 * (lane % QCH);
#pragma unroll
      for (int i = 0; i < QI; ++i) {
        const int row = lane / QCH + (64 / QCH) * i;
        const float dzr = dzs[32 + row];
        const u32x4 w{pack2<T>(dzr * kmc[0], dzr * kmc[1]), pack2<T>(dzr * kmc[2], dzr * kmc[3]),
                      pack2<T>(dzr * kmc[4], dzr * kmc[5]), pack2<T>(dzr * kmc[6], dzr * kmc[7])};
        const int64_t off = piece(t0 + row, lane % QCH, dk);
        if (off >= 0) store_row16<kNtPassAStore>(dqd + off, w);
      }
    }
    t0 = tn;
  }

  if constexpr (FUSED) {
    __syncthreads();  // every wave is done with its tiles: reuse them for the reduction
    float* red = reinterpret_cast<float*>(smem + LY::kOpnd);
    float* dst = fin_mat ? fin_mat + (int64_t)nh * dk * dv
                         : partial + partial_slot(p, n, h, c, nchunks) * (dk * dv + dk);
    float* dst_vec = fin_mat ? (fin_vec ? fin_vec + (int64_t)nh * dk : nullptr) : dst + dk * dv;
    const float mscale = fin_mat ? seq_scale(p, len) : 1.f;
    const float vscale = fin_mat ? 1.0f / (float)len : 1.f;
    reduce_store_block<4, true, PAIR>(acc, dkm, red, dst, dv, dst_vec, mscale, vscale, wave, lane, dk, dv);
  }
}

// ===========================================================================
// backward pass A, heads tiled 128 x 128
// ===========================================================================
// dS (128 x 128 fp32) does not fit one wave, so a workgroup of four waves shares steps of 64
// tokens (two 32-token tiles) and two workgroups share a CU, each filling the other's waits:
//   prologue      the S^T operand (hi + lo, 64 KiB) is built in LDS once; wave w keeps the
//                 fragments of output block w (32 of the 128 columns of g = dO S^T) in 64
//                 registers, and the LDS they were built in becomes the tiles;
//   token view    wave w multiplies both tiles by its block, adds its part of q~.g and q.km; the
//                 four parts of a token meet in LDS, then every wave knows 1/z_t and dz_t, packs
//                 its 32 columns of dq into a staging tile (whole rows leave from there) and
//                 scales its quarter of the dO tile by 1/z_t into a hi and a lo tile, once for
//                 all waves;
//   feature view  wave w owns 64 x 64 block w of dS; q~^T and dO / z come straight out of the
//                 row-major tiles in operand order through the transposing LDS read
//                 (ds_read_b64_tr_b16: a lane receives four tokens of one feature), so there
//                 is no in-register transposition and no rescaling here.
// The contraction index of the feature view is a permutation of the tile's tokens (the same for
// both operands): k-step ks, half-wave kb, element e = 4x + j is token 16ks + 4j + 2kb + x.  One
// transposing read then touches four token rows that differ in bits 2..3, which the XOR swizzle
// of the tiles spreads over all banks.
struct BwdA128Layout {
  static constexpr int kOpnd = 4 * 8 * 2 * 1024;  // 4 blocks x 8 k-steps x (hi, lo) fragments
  static constexpr int kTile = 32 * 256;          // 32 tokens x 128 features x 2 bytes
  static constexpr int kQ = 0;                    // q tiles [2]
  static constexpr int kG = kQ + 2 * kTile;       // dO tiles [2], then the hi part of dO / z
  static constexpr int kGl = kG + 2 * kTile;      // lo part of dO / z
  static constexpr int kDq = kGl + 2 * kTile;     // dq staging [2]
  static constexpr int kPz = kDq + 2 * kTile;     // [tile][block][32] partial (q~.g, q.km)
  static constexpr int kDz = kPz + 2 * 4 * 32 * 8;  // [hi, lo][tile] dz in contraction order, 16-bit
  static constexpr int kKmPairs = kDz + 2 * 32 * 4;
  static constexpr int kKmF = kKmPairs + 128 * 4;
  static constexpr int kMax = kKmF + 128 * 4;
  static constexpr int kLpt = kMax + 64;
  static constexpr int kTotal = kLpt + (kLptMax + 1) * 4;
  static_assert(kPz >= kOpnd, "the operand is built where the tiles will be");
  static_assert(2 * kTotal <= 160 * 1024, "two workgroups per CU");
};

template <typename T, bool NORM, bool PAD>
__global__ __launch_bounds__(256, 2) void bwd_a128_kernel(
    Prob p, const T* __restrict__ qn, const T* __restrict__ dout, const float* __restrict__ S,
    const float* __restrict__ km, T* __restrict__ dqn, float* __restrict__ partial, float* fin_mat,
    float* fin_vec, int chunk, int nchunks) {
  using LY = BwdA128Layout;
  constexpr bool LO = !std::is_same<T, _Float16>::value;  // see launch_bwd_a
  constexpr int KS = 8, ROWB = 256, NT = 256;
  const int dk = PAD ? p.DK : 128, dv = PAD ? p.DV : 128;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

  const int wg_item = packed_item(p, blockIdx.x, p.H * nchunks);
  const int wg_nh = wg_item / nchunks, c = wg_item - wg_nh * nchunks;
  const int h = wg_nh % p.H;
  const int n = lpt_sequence(p, wg_nh / p.H, reinterpret_cast<int*>(smem + LY::kLpt));
  const int nh = n * p.H + h;
  int64_t bos, row0, rstride;
  int len;
  seq_range(p, n, bos, len);
  const int t_begin = c * chunk;
  if (t_begin >= len) {
    if (fin_mat && c == 0) {  // empty sequence: no gradient flows through its state
      for (int e = threadIdx.x; e < dk * dv; e += NT) fin_mat[(int64_t)nh * dk * dv + e] = 0.f;
      if (fin_vec)
        for (int e = threadIdx.x; e < dk; e += NT) fin_vec[(int64_t)nh * dk + e] = 0.f;
    }
    return;
  }
  const int t_end = min(len, t_begin + chunk);
  row_base(p, n, h, bos, row0, rstride);

  const int tid = threadIdx.x, blk = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int ntok = lane & 31, kb = lane >> 5;
  const int bk = blk >> 1, bv = blk & 1;  // feature view: block (bk, bv) of dS
  unsigned char* qtile = smem + LY::kQ;
  unsigned char* gtile = smem + LY::kG;
  unsigned char* gltile = smem + LY::kGl;
  unsigned char* dqtile = smem + LY::kDq;
  float* pz = reinterpret_cast<float*>(smem + LY::kPz);
  T* dzp = reinterpret_cast<T*>(smem + LY::kDz);  // [hi, lo][tile][32]
  uint32_t* km_pairs = reinterpret_cast<uint32_t*>(smem + LY::kKmPairs);
  float* kmf = reinterpret_cast<float*>(smem + LY::kKmF);
  float* lds_max = reinterpret_cast<float*>(smem + LY::kMax);

  // The workgroup moves the 1024 16-byte pieces of a step's 64 rows: thread t takes pieces
  // t + 256 i, i.e. chunk t % 16 of rows t / 16 + 16 i.  A piece's address is the step's uniform
  // address plus a uniform i-th distance plus the lane's one constant byte offset (32 bits: the
  // host keeps packed tensors with more than 65536 heads away from this kernel).
  const int prow = tid >> 4, pch = tid & 15;
  const uint32_t qrow_b = (uint32_t)rstride * (uint32_t)dk * 2u, grow_b = (uint32_t)rstride * (uint32_t)dv * 2u;
  const uint32_t qvoff = (uint32_t)prow * qrow_b + (uint32_t)pch * 16u;
  const uint32_t gvoff = PAD ? (uint32_t)prow * grow_b + (uint32_t)pch * 16u : qvoff;
  const bool q_piece = !PAD || pch * 8 < dk, g_piece = !PAD || pch * 8 < dv;  // the chunk exists in a row
  auto step_ptr = [&](const void* src, int tok0, int rowlen) -> const char* {
    return reinterpret_cast<const char*>(src) + ((row0 + (int64_t)tok0 * rstride) * rowlen) * (int64_t)sizeof(T);
  };
  auto load_step = [&](u32x4(&dst)[4], const T* src, int tok0, int rowlen, uint32_t row_b, uint32_t voff, bool has) {
    const char* tp = step_ptr(src, tok0, rowlen);
    const int rows = t_end - tok0;  // rows of this step that exist (may be <= 0)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      dst[i] = u32x4{0u, 0u, 0u, 0u};
      if (has && prow + 16 * i < rows) dst[i] = load_stream<u32x4, kNtPassALoad>(tp + (size_t)(16 * i) * row_b + voff);
    }
  };
  auto stash_step = [&](const u32x4(&src)[4], unsigned char* tiles) {
#pragma unroll
    for (int i = 0; i < 4; ++i) *reinterpret_cast<u32x4*>(tiles + swz<ROWB>(prow + 16 * i, pch)) = src[i];
  };

  f32x16 acc[2][2];
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.f;
  float dkm = 0.f;  // row 64 bk + 32 bv + ntok, this half-wave's tokens

  u32x4 rq[4], rg[4];
  load_step(rq, qn, t_begin, dk, qrow_b, qvoff, q_piece);
  load_step(rg, dout, t_begin, dv, grow_b, gvoff, g_piece);

  // g_t = dO_t S^T: contraction over dv, M(r = dv, c = dk) = S[c][r]
  const float denorm = build_operand<T, 128, 128, NT, PAD>(smem, lds_max, S + (int64_t)nh * dk * dv, 1, dv, 1, 0,
                                                          1.f, nullptr, dv, dk);
  if constexpr (NORM) build_vec<T, NT>(km_pairs, kmf, km + (int64_t)nh * dk, dk, 1, 0, 1.f, nullptr, 128);
  __syncthreads();
  u32x4 sh[KS], sl[KS];  // output block blk: columns 64 kb' + 16 blk + 0..15 of lane (token, kb')
#pragma unroll
  for (int s = 0; s < KS; ++s) {
    const int f = blk * KS + s;
    sh[s] = *reinterpret_cast<const u32x4*>(smem + ((2 * f + 0) * 64 + lane) * 16);
    sl[s] = *reinterpret_cast<const u32x4*>(smem + ((2 * f + 1) * 64 + lane) * 16);
  }
  __syncthreads();  // the operand has left LDS

  // transposing reads: this lane addresses, for element half x, token 4 (s >> 2) + 2 (g >> 1) + x
  // (+ 16 ks) and the four features 16 (g & 1) + 4 (s & 3) .. + 3 of the fragment (g = lane / 16,
  // s = lane % 16)
  int qoff[2][2], goff[2][2];
  {
    const int g16 = lane >> 4, s16 = lane & 15;
#pragma unroll
    for (int x = 0; x < 2; ++x) {
      const int tok = 4 * (s16 >> 2) + 2 * (g16 >> 1) + x;
      const int f0 = 16 * (g16 & 1) + 4 * (s16 & 3);
#pragma unroll
      for (int a = 0; a < 2; ++a) {
        const int fq = 64 * bk + 32 * a + f0, fg = 64 * bv + 32 * a + f0;
        qoff[a][x] = swz<ROWB>(tok, fq >> 3) + ((fq >> 2) & 1) * 8;
        goff[a][x] = swz<ROWB>(tok, fg >> 3) + ((fg >> 2) & 1) * 8;
      }
    }
  }
  // position of token ntok in the contraction order of its tile
  const int kpos = (ntok & 16) | ((ntok & 2) << 2) | ((ntok & 1) << 2) | ((ntok >> 2) & 3);

  for (int base = t_begin; base < t_end; base += 64) {
    stash_step(rq, qtile);
    stash_step(rg, gtile);
    __syncthreads();

    // ---- token view: this lane gets columns 64 kb + 16 blk + 0..15 of token ntok of both tiles
    f32x16 g[2];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
#pragma unroll
      for (int r = 0; r < 16; ++r) g[t][r] = 0.f;
#pragma unroll
      for (int s = 0; s < KS; ++s) {
        const u32x4 bq = *reinterpret_cast<const u32x4*>(gtile + t * LY::kTile + swz<ROWB>(ntok, KS * kb + s));
        g[t] = Ops<T>::mma(sh[s], bq, g[t]);
        g[t] = Ops<T>::mma(sl[s], bq, g[t]);
      }
    }
    // the next step's rows are requested here, not at the top of the step: their 32 registers are
    // then free during the token view, whose LDS reads need buffers to be in flight ahead of the products
    load_step(rq, qn, base + 64, dk, qrow_b, qvoff, q_piece);
    load_step(rg, dout, base + 64, dv, grow_b, gvoff, g_piece);
    float rz[2] = {1.f, 1.f}, dz[2] = {0.f, 0.f};
    if constexpr (NORM) {
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        float P = 0.f, z = 0.f;
#pragma unroll
        for (int ch = 0; ch < 2; ++ch) {
          const u32x4 qw =
              *reinterpret_cast<const u32x4*>(qtile + t * LY::kTile + swz<ROWB>(ntok, 8 * kb + 2 * blk + ch));
          const u32x4 kh = *reinterpret_cast<const u32x4*>(&km_pairs[32 * kb + 8 * blk + 4 * ch]);
          const u32x4 kl = *reinterpret_cast<const u32x4*>(&km_pairs[64 + 32 * kb + 8 * blk + 4 * ch]);
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const int c0 = 8 * ch + 2 * i;
            P = fmaf(Ops<T>::lo(qw[i]), g[t][c0], P);
            P = fmaf(Ops<T>::hi(qw[i]), g[t][c0 + 1], P);
            z = Ops<T>::dot2(qw[i], kh[i], z);
            z = Ops<T>::dot2(qw[i], kl[i], z);
          }
        }
        P = sum_halves(P);
        z = sum_halves(z);
        if (kb == 0) *reinterpret_cast<float2*>(&pz[2 * ((4 * t + blk) * 32 + ntok)]) = float2{P, z};
      }
      __syncthreads();
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        float P = 0.f, z = 0.f;  // the four parts in block order: the same sum in every wave
#pragma unroll
        for (int b = 0; b < 4; ++b) {
          const float2 part = *reinterpret_cast<const float2*>(&pz[2 * ((4 * t + b) * 32 + ntok)]);
          P += part.x;
          z += part.y;
        }
        if (base + 32 * t + ntok < t_end) {
          rz[t] = 1.f / (z + p.eps);
          dz[t] = -(P * denorm) * rz[t] * rz[t];
        } else {
          rz[t] = 0.f;  // padding rows contribute nothing
        }
        if (blk == 0 && kb == 0) {  // dz as a 16-bit hi + lo pair, for the dot products of the feature view
          const T dh = (T)dz[t], dl = (T)(dz[t] - (float)dh);
          dzp[32 * t + kpos] = dh;
          dzp[64 + 32 * t + kpos] = dl;
        }
      }
    }
    // dq: this wave's 32 columns of every row, into the staging tiles
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const float gs = denorm * rz[t];
#pragma unroll
      for (int ch = 0; ch < 2; ++ch) {
        u32x4 w;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int c0 = 8 * ch + 2 * i;
          float v0 = g[t][c0] * gs, v1 = g[t][c0 + 1] * gs;
          if constexpr (NORM) {
            v0 = fmaf(dz[t], kmf[64 * kb + 16 * blk + c0], v0);
            v1 = fmaf(dz[t], kmf[64 * kb + 16 * blk + c0 + 1], v1);
          }
          w[i] = pack2<T>(v0, v1);
        }
        *reinterpret_cast<u32x4*>(dqtile + t * LY::kTile + swz<ROWB>(ntok, 8 * kb + 2 * blk + ch)) = w;
      }
    }
    // dO / z as hi + lo: this wave's quarter of every row (chunks 4 blk + 2 kb + 0..1)
    if constexpr (NORM) {
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int ch = 0; ch < 2; ++ch) {
          const int off = t * LY::kTile + swz<ROWB>(ntok, 4 * blk + 2 * kb + ch);
          const u32x4 gw = *reinterpret_cast<const u32x4*>(gtile + off);
          u32x4 wh, wl;
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const float a = Ops<T>::lo(gw[i]) * rz[t], b = Ops<T>::hi(gw[i]) * rz[t];
            const T ah = (T)a, bh = (T)b;
            wh[i] = pack2<T>((float)ah, (float)bh);
            if constexpr (LO) wl[i] = pack2<T>(a - (float)ah, b - (float)bh);
          }
          *reinterpret_cast<u32x4*>(gtile + off) = wh;
          if constexpr (LO) *reinterpret_cast<u32x4*>(gltile + off) = wl;
        }
    }
    __syncthreads();  // dq rows, dO / z and dz are complete

    {
      char* tp = const_cast<char*>(step_ptr(dqn, base, dk));
      const int rows = t_end - base;
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (q_piece && prow + 16 * i < rows)
          store_row16<kNtPassAStore>(tp + (size_t)(16 * i) * qrow_b + qvoff,
                                     *reinterpret_cast<const u32x4*>(dqtile + swz<ROWB>(prow + 16 * i, pch)));
    }

    // ---- feature view: dS block (bk, bv) += q~^T (dO / z) over both tiles
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int ks = 0; ks < 2; ++ks) {
        const int tb = t * LY::kTile + ks * 16 * ROWB;
        u32x4 A[2], Bh[2];
#pragma unroll
        for (int a = 0; a < 2; ++a) {
          A[a] = tr_fragment(qtile + tb, qoff[a][0], qoff[a][1]);
          Bh[a] = tr_fragment(gtile + tb, goff[a][0], goff[a][1]);
        }
#pragma unroll
        for (int a = 0; a < 2; ++a)
#pragma unroll
          for (int b = 0; b < 2; ++b) acc[a][b] = Ops<T>::mma(A[a], Bh[b], acc[a][b]);
        if constexpr (NORM) {
          if constexpr (LO) {
            u32x4 Bl[2];
#pragma unroll
            for (int b = 0; b < 2; ++b) Bl[b] = tr_fragment(gltile + tb, goff[b][0], goff[b][1]);
#pragma unroll
            for (int a = 0; a < 2; ++a)
#pragma unroll
              for (int b = 0; b < 2; ++b) acc[a][b] = Ops<T>::mma(A[a], Bl[b], acc[a][b]);
          }
          // dkm of the rows of A[bv] (the two waves of a key half share its 64 rows)
          const u32x4 Ad = bv ? A[1] : A[0];
          const T* dzs = dzp + 32 * t + 16 * ks + 8 * kb;
          const u32x4 dh = *reinterpret_cast<const u32x4*>(dzs), dl = *reinterpret_cast<const u32x4*>(dzs + 64);
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            dkm = Ops<T>::dot2(Ad[i], dh[i], dkm);
            dkm = Ops<T>::dot2(Ad[i], dl[i], dkm);
          }
        }
      }
    __syncthreads();  // every wave has read the tiles: the next step may take their place
  }

  {
    float* dst = fin_mat ? fin_mat + (int64_t)nh * dk * dv
                         : partial + partial_slot(p, n, h, c, nchunks) * (dk * dv + dk);
    float* dst_vec = fin_mat ? (fin_vec ? fin_vec + (int64_t)nh * dk : nullptr) : dst + dk * dv;
    const float mscale = fin_mat ? seq_scale(p, len) : 1.f;
    const float vscale = fin_mat ? 1.0f / (float)len : 1.f;
    float none[2] = {0.f, 0.f};
    reduce_store_block<1, false>(acc, none, nullptr, dst + (64 * bk) * dv + 64 * bv, dv, nullptr, mscale, vscale, 0,
                                 lane, dk - 64 * bk, dv - 64 * bv);
    const float tot = dkm + __shfl_xor(dkm, 32);
    const int row = 64 * bk + 32 * bv + ntok;
    if (dst_vec && kb == 0 && row < dk) dst_vec[row] = NORM ? tot * vscale : 0.f;
  }
}

// ===========================================================================
// host side
// ===========================================================================
// The kernels tile a head into 64-wide blocks: a head dim runs as the next of 64 / 128 above
// it, the padded variants (PAD) when it is not one of the two.
static int tiled_dim(int d) { return d <= 64 ? 64 : 128; }
static bool padded(const Prob& p) { return p.DK != tiled_dim(p.DK) || p.DV != tiled_dim(p.DV); }

// Dense tensors with 32 x 32 heads: the row-parallel kernels take two tokens per 64-wide row
// (PAIR variants) instead of padding every row to 64.
bool pair_mode(const Prob& p, int dtype) {
  return (dtype == kF16 || dtype == kBF16) && !p.cu && p.DK == 32 && p.DV == 32;
}

// 16-bit inputs with head dims that are multiples of 8 (16-byte row pieces) up to 128.
bool supported(const Prob& p, int dtype) {
  if (dtype == kF32) return mfma32::supported(p);
  if (dtype != kF16 && dtype != kBF16) return false;
  if (p.DK < 8 || p.DV < 8 || p.DK > 128 || p.DV > 128 || p.DK % 8 || p.DV % 8) return false;
  return true;
}

// The fused backward pass A exists for heads tiled as 64 x 64 and as 128 x 128 (the latter
// not for the decoupled operator).
static int knob(const char* name, int dflt);
bool bwd_a_supported(const Prob& p, int dtype) {
  if (dtype == kF32 || !supported(p, dtype)) return false;
  const bool wide = tiled_dim(p.DK) == 128 || tiled_dim(p.DV) == 128;
  // heads with one 128-wide side run as padded 128 x 128 heads of the plain operator (one pass over
  // q and dO instead of two)
  static const bool mixed = knob("FBLA_BWDA_MIXED", 1) == 1;
  if (tiled_dim(p.DK) != tiled_dim(p.DV) && ((p.flags & kDecoupled) || !mixed)) return false;
  // the 128 x 128 kernel addresses a step's rows with 32-bit lane offsets
  if (wide && p.cu && p.H > 65536) return false;
  // decoupled: fused for 64 x 64 tiles only (the 128 x 128 kernel has no room for the plain q tile)
  return !(p.flags & kDecoupled) || !wide;
}

// Number of compute units of the current device (256 on MI355X; also the value
// assumed when no device is visible, e.g. for a host-only workspace query).
static int cu_count() {
  static const int n = [] {
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) {
      (void)hipGetLastError();
      return 256;
    }
    return cus;
  }();
  return n;
}

// Integer tuning constant (environment override only in -DFBLA_TUNING builds).
static int knob(const char* name, int dflt) { return tuning_knob(name, dflt); }

// Tokens per workgroup for a kernel of which `wgs_per_cu` workgroups fit on a CU:
// the grid is sized to at most `rounds` full rounds of resident workgroups, with
// all workgroups doing the same amount of work (no ragged last round).
// Packed batches: the grid is laid out for the longest sequence, so a batch with one very
// long sequence among short ones would leave that sequence to one workgroup per head.  When
// the longest sequence is more than four times a workgroup's fair share of all tokens, the
// chunk shrinks to twice that share (the workgroups of the chunks a short sequence does not
// have exit at once).  `reduction`: the kernel writes a partial per chunk, whose storage grows
// with the number of chunks of the longest sequence times all (sequence, head) pairs: the
// number of chunks is then also kept within 1 GiB of partials (reserved, only the chunks
// that exist are written and read) and 64.
static int chunk_for(const Prob& p, int wgs_per_cu, int rounds, int min_chunk, int align, bool reduction) {
  const int64_t nh = (int64_t)p.N * p.H;
  const int64_t slots = (int64_t)cu_count() * wgs_per_cu * rounds;
  int64_t nchunks = slots / (nh > 0 ? nh : 1);
  if (nchunks < 1) nchunks = 1;
  int64_t chunk = cdiv64(p.L, nchunks);
  if (p.cu && nh > 0) {
    const int64_t fair = cdiv64(p.T * p.H, slots);
    if (p.L > 4 * fair && chunk > 2 * fair) {
      chunk = 2 * fair;
      if (reduction) {
        const int64_t level_bytes = nh * ((int64_t)p.DK * p.DV + p.DK) * (int64_t)sizeof(float);
        int64_t levels = (1LL << 30) / (level_bytes > 0 ? level_bytes : 1);
        levels = levels < 1 ? 1 : (levels > 64 ? 64 : levels);
        if (chunk < cdiv64(p.L, levels)) chunk = cdiv64(p.L, levels);
      }
    }
  }
  if (chunk < min_chunk) chunk = min_chunk;
  chunk = cdiv64(chunk, align) * align;
  return (int)chunk;
}

// Reduction kernels (state, backward pass A): one round of resident workgroups.
// 128 x 128 states of the plain operator: state128_kernel, two workgroups per CU.
static int whole_state_chunk(const Prob& p) {
  static const int on = knob("FBLA_STATE128", 1);  // 2 = off (A/B comparisons)
  if (on != 1 || tiled_dim(p.DK) != 128 || tiled_dim(p.DV) != 128 || (p.flags & kDecoupled)) return 0;
  if (p.cu && p.H > 65536) return 0;  // 32-bit lane offsets
  return chunk_for(p, 2, 1, 256, 64, true);
}

// Dense heads short enough for one workgroup each: the state kernel stores the finished sums itself (no
// partials, no reduce launch) when that leaves at least a quarter of the CUs with a workgroup.
// B8-H16-D64 fp16 forward: T=512 21.8 -> 20.3 us, T=1024 28.2 -> 25.9 us, T=2048 41.1 -> 40.7 us; backward
// pass A loses with it (step as a HIP graph at T=1024 71.1 -> 72.0 us, at T=2048 107 -> 115 us) and keeps its chunks.
static int whole_sequence_chunk(const Prob& p, int align) {
  static const int max_len = knob("FBLA_DIRECT_MAX_L", 1024);
  if (p.cu || p.L > max_len || (int64_t)p.N * p.H * 4 < cu_count()) return 0;
  return (int)(cdiv64(p.L, align) * align);
}

int state_chunk(const Prob& p, bool block_stats) {
  static const int per_cu = knob("FBLA_STATE_WGS_PER_CU", 2);
  if (!block_stats) {
    const int direct = whole_sequence_chunk(p, 64);
    if (direct) return direct;
  }
  const int whole = block_stats && padded(p) ? 0 : whole_state_chunk(p);
  return whole ? whole : chunk_for(p, per_cu, 1, 256, 64, true);
}

int bwd_a_chunk(const Prob& p) {
  static const int per_cu = knob("FBLA_BWDA_WGS_PER_CU", 2);

  // 128 x 128: two workgroups of four waves per CU, steps of 64 tokens
  if (tiled_dim(p.DK) == 128 || tiled_dim(p.DV) == 128) return chunk_for(p, 2, 1, 512, 64, true);
  return chunk_for(p, per_cu, 1, 256, 128, true);
}

static bool use_rows128(const Prob& p);
// Row-parallel kernels: long enough chunks to amortise the operand prologue.
int rows_chunk(const Prob& p, int DR, int DC) {
  static const int per_cu_knob = knob("FBLA_ROWS_WGS_PER_CU", 4);
  // dense: several rounds of short workgroups (page locality); packed: one workgroup per
  // (sequence, head) where possible, handed out longest first, so fewer operand prologues
  static const int dense_rounds = knob("FBLA_ROWS_ROUNDS", 4);
  static const int packed_rounds = knob("FBLA_ROWS_ROUNDS_PACKED", 1);
  // a 128 x 128 operand costs as much to build as 512 tokens cost to stream: one round there
  const int big = (tiled_dim(DR) == 128) + (tiled_dim(DC) == 128);
  const int per_cu = big == 0 ? per_cu_knob : (big == 1 || use_rows128(p) ? 2 : 1);
  // (one 128-wide side: half the operand, still one round - B8-H16-T4096 fp16 fwd+bwd with two rounds
  // DK128-DV64 0.304 against 0.298 ms, DK96-DV48 0.277 against 0.265 ms)
  static const int rect_rounds = knob("FBLA_ROWS_ROUNDS_RECT", 1);
  int rounds = p.cu ? packed_rounds : (big == 2 ? 1 : big == 1 ? rect_rounds : dense_rounds);
  // packed batches of 64-wide tiles whose lengths are of one order (not the one-long-among-short
  // case that chunk_for treats by itself): up to three chunks per sequence, so that the longest
  // sequences, which start first, do not each keep one workgroup busy to the end (64 sequences of
  // 256..2048 tokens, H16-D64: forward output 84 -> 75 us, forward + backward 0.427 -> 0.404 ms)
  static const int even_rounds = knob("FBLA_ROWS_ROUNDS_PACKED_EVEN", 3);
  if (p.cu && big == 0 && rounds < even_rounds) {
    const int64_t fair = cdiv64(p.T * p.H, (int64_t)cu_count() * per_cu * rounds);
    if (p.L <= 4 * fair) rounds = even_rounds;
  }
  static const int min_chunk_knob = knob("FBLA_ROWS_MIN_CHUNK", 256);
  // a problem too small to give every CU a workgroup: shorter chunks (the operand build of the
  // extra workgroups costs less than the idle CUs)
  int min_chunk = min_chunk_knob;
  const int64_t nh = (int64_t)p.N * p.H;
  while (min_chunk > 128 && big < 2 && nh * cdiv64(p.L, min_chunk) < cu_count()) min_chunk /= 2;
  int chunk = chunk_for(p, per_cu, rounds, min_chunk, big == 2 ? 256 : 128, false);
  // dense 64-wide tiles: no more than 512 tokens per workgroup however long the sequences are
  // (more, shorter workgroups balance better than four rounds of long ones: B8-H16-T32768 fwd+bwd
  // 1.160 -> 1.126 ms)
  static const int max_chunk = knob("FBLA_ROWS_MAX_CHUNK", 512);
  if (!p.cu && big == 0 && chunk > max_chunk && max_chunk >= min_chunk) chunk = max_chunk;
  return chunk;
}

// Reserves the kernel's dynamic LDS once per instantiation and thread.
template <typename K> static int reserve_lds(K kernel, int bytes, bool& done) {
  if (done) return kOk;
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
  if (e != hipSuccess) {
    set_error("cannot reserve %d bytes of LDS: %s", bytes, hipGetErrorString(e));
    return kErrLaunch;
  }
  done = true;
  return kOk;
}

template <typename T, int DK, int DV, bool PAD>
static void launch_state(const Prob& p, const T* kn, const T* v, const T* kd, float* partial,
                         const float* tokscal, int64_t total_rows, float* fm, float* fv, int chunk,
                         int nchunks, BlockStats bs, hipStream_t st) {
  const dim3 grid((unsigned)((int64_t)p.N * p.H * nchunks)), block(kThreads);
  // 16-token tiles per step and wave: two for the 128 x 128 state, whose waves all walk the
  // same tokens and so have half as many bytes in flight per token (packed batches with a
  // few long sequences finish 9 % sooner)
  constexpr int TL = (DK == 128 && DV == 128) ? 2 : 1;
  if constexpr (DK == 128 && DV == 128) {
    if (!tokscal && whole_state_chunk(p) == chunk && !(bs.kc && PAD)) {
      static thread_local bool configured[2] = {false, false};  // per instantiation
      if (bs.kc) {
        if constexpr (!PAD) {
          auto kernel = state128_kernel<T, false, true>;
          if (reserve_lds(kernel, State128Layout::kTotal, configured[1]) != kOk) return;
          kernel<<<grid, block, State128Layout::kTotal, st>>>(p, kn, v, partial, fm, fv, chunk, nchunks, bs);
        }
      } else {
        auto kernel = state128_kernel<T, PAD>;
        if (reserve_lds(kernel, State128Layout::kTotal, configured[0]) != kOk) return;
        kernel<<<grid, block, State128Layout::kTotal, st>>>(p, kn, v, partial, fm, fv, chunk, nchunks, bs);
      }
      return;
    }
  }
  if (p.flags & kElu1) {  // (the plan has checked: 64 x 64, plain operator)
    if constexpr (DK == 64 && DV == 64 && !PAD)
      state_kernel<T, 64, 64, false, 1, false, false, false, true><<<grid, block, 0, st>>>(p, kn, v, kd, partial, nullptr, 0, fm, fv, chunk, nchunks, bs);
  } else if (bs.kc) {
    if constexpr (!PAD)
      state_kernel<T, DK, DV, false, 1, false, true><<<grid, block, 0, st>>>(p, kn, v, kd, partial, nullptr, 0, fm, fv, chunk, nchunks, bs);
  } else if (tokscal && (p.flags & kDecoupled))  // dkm = sum_t dz_t q_t over the plain q rows (kd)
    state_kernel<T, DK, DV, true, 1, true, false, PAD><<<grid, block, 0, st>>>(p, kn, v, kd, partial, tokscal, total_rows, fm, fv, chunk, nchunks, bs);
  else if (tokscal)
    state_kernel<T, DK, DV, false, 1, true, false, PAD><<<grid, block, 0, st>>>(p, kn, v, kd, partial, tokscal, total_rows, fm, fv, chunk, nchunks, bs);
  else if (p.flags & kDecoupled)
    state_kernel<T, DK, DV, true, TL, false, false, PAD><<<grid, block, 0, st>>>(p, kn, v, kd, partial, nullptr, 0, fm, fv, chunk, nchunks, bs);
  else
    state_kernel<T, DK, DV, false, TL, false, false, PAD><<<grid, block, 0, st>>>(p, kn, v, kd, partial, nullptr, 0, fm, fv, chunk, nchunks, bs);
}

template <typename T, bool PAD>
static void run_state_dims(const Prob& p, const T* a, const T* b, const T* c, float* partial,
                           const float* ts, int64_t rows, float* fm, float* fv, int chunk, int nchunks,
                           BlockStats bs, hipStream_t st) {
  const int DK = tiled_dim(p.DK), DV = tiled_dim(p.DV);
  if (DK == 64 && DV == 64) launch_state<T, 64, 64, PAD>(p, a, b, c, partial, ts, rows, fm, fv, chunk, nchunks, bs, st);
  else if (DK == 64) launch_state<T, 64, 128, PAD>(p, a, b, c, partial, ts, rows, fm, fv, chunk, nchunks, bs, st);
  else if (DV == 64) launch_state<T, 128, 64, PAD>(p, a, b, c, partial, ts, rows, fm, fv, chunk, nchunks, bs, st);
  else launch_state<T, 128, 128, PAD>(p, a, b, c, partial, ts, rows, fm, fv, chunk, nchunks, bs, st);
}

template <typename T>
static void run_state(const Prob& p, const void* kn, const void* v, const void* kd, float* partial,
                      const float* ts, int64_t rows, float* fm, float* fv, int chunk, int nchunks,
                      BlockStats bs, hipStream_t st) {
  const T *a = (const T*)kn, *b = (const T*)v, *c = (const T*)kd;
  if (padded(p)) run_state_dims<T, true>(p, a, b, c, partial, ts, rows, fm, fv, chunk, nchunks, bs, st);
  else run_state_dims<T, false>(p, a, b, c, partial, ts, rows, fm, fv, chunk, nchunks, bs, st);
}

template <typename T, int DR, int DC, bool NORM, bool DEN, int WAVES, bool PAD, bool PAIR = false, bool FMAP = false,
          bool GATE = false>
static int launch_rows_k(const Prob& p, const RowsJob& job, const RowsJob* job2, int chunk,
                         int nchunks, int dr, int dc, hipStream_t st) {
  using LY = RowsLayout<DR, DC, DEN, WAVES, GATE>;
  constexpr int PF = (DR == 128 && DC == 128) ? FBLA_ROWS_PF128 : FBLA_ROWS_PF;
  auto kernel = rows_kernel<T, DR, DC, NORM, DEN, WAVES, PAD, PF, PAIR, FMAP, GATE>;
  static thread_local bool configured = false;
  int rc = reserve_lds(kernel, LY::kTotal, configured);
  if (rc != kOk) return rc;
  const int wgs = (int)((int64_t)p.N * p.H * nchunks);
  const dim3 grid((unsigned)(job2 ? 2 * wgs : wgs)), block(WAVES * 64);
  kernel<<<grid, block, LY::kTotal, st>>>(p, job, job2 ? *job2 : job, wgs, chunk, nchunks, dr, dc);
  return kOk;
}

template <typename T, bool NORM, bool PAD>
static int launch_rows128(const Prob& p, const RowsJob& job, const RowsJob* job2, int chunk, int nchunks, int dr,
                          int dc, hipStream_t st) {
  auto kernel = rows128_kernel<T, NORM, PAD>;
  static thread_local bool configured = false;
  int rc = reserve_lds(kernel, Rows128Layout::kTotal, configured);
  if (rc != kOk) return rc;
  const int wgs = (int)((int64_t)p.N * p.H * nchunks);
  const dim3 grid((unsigned)(job2 ? 2 * wgs : wgs)), block(kThreads);
  kernel<<<grid, block, Rows128Layout::kTotal, st>>>(p, job, job2 ? *job2 : job, wgs, chunk, nchunks, dr, dc);
  return kOk;
}

// 128 x 128 matrices without separate denominator rows: rows128_kernel (FBLA_ROWS128=2 keeps the
// general kernel, for comparisons)
static bool use_rows128(const Prob& p) {
  static const int on = knob("FBLA_ROWS128", 1);
  return on == 1 && !(p.flags & kDecoupled) && !(p.cu && p.H > 65536);
}

template <typename T, int DR, int DC, bool PAD>
static int launch_rows(const Prob& p, const RowsJob& job, const RowsJob* job2, int dr, int dc,
                       hipStream_t st) {
  // 128 x 128 operands fill 64 KiB of LDS: one 8-wave workgroup per CU instead of
  // several 4-wave ones
  constexpr int WAVES = (DR == 128 && DC == 128) ? 8 : 4;
  const int chunk = rows_chunk(p, DR, DC);
  const int nchunks = (int)cdiv64(p.L, chunk);
  const bool norm = job.xden != nullptr;
  const bool den = norm && job.xden != job.x;
  if constexpr (DR == 128 && DC == 128) {
    if (!den && use_rows128(p)) {
      if (norm) return launch_rows128<T, true, PAD>(p, job, job2, chunk, nchunks, dr, dc, st);
      return launch_rows128<T, false, PAD>(p, job, job2, chunk, nchunks, dr, dc, st);
    }
  }
  if constexpr (DR == 64 && DC == 64 && !PAD) {
    if (job.gate || (job2 && job2->gate)) {  // (the plan has checked: pass B of the plain operator)
      if (p.flags & kElu1)  // keys before the map
        return launch_rows_k<T, 64, 64, false, false, WAVES, false, false, true, true>(p, job, job2, chunk, nchunks, dr, dc, st);
      return launch_rows_k<T, 64, 64, false, false, WAVES, false, false, false, true>(p, job, job2, chunk, nchunks, dr, dc, st);
    }
    if (p.flags & kElu1) {  // (the plan has checked: plain operator, forward output)
      if (norm) return launch_rows_k<T, 64, 64, true, false, WAVES, false, false, true>(p, job, job2, chunk, nchunks, dr, dc, st);
      return launch_rows_k<T, 64, 64, false, false, WAVES, false, false, true>(p, job, job2, chunk, nchunks, dr, dc, st);
    }
  }
  if (!norm) return launch_rows_k<T, DR, DC, false, false, WAVES, PAD>(p, job, job2, chunk, nchunks, dr, dc, st);
  if (!den) return launch_rows_k<T, DR, DC, true, false, WAVES, PAD>(p, job, job2, chunk, nchunks, dr, dc, st);
  return launch_rows_k<T, DR, DC, true, true, WAVES, PAD>(p, job, job2, chunk, nchunks, dr, dc, st);
}

// two tokens per row: chunks are counted in row pairs
template <typename T>
static int launch_rows_pair(const Prob& p, const RowsJob& job, const RowsJob* job2, hipStream_t st) {
  Prob pw = p;
  pw.L = (p.L + 1) / 2;
  const int chunk = rows_chunk(pw, 64, 64);
  const int nchunks = (int)cdiv64(pw.L, chunk);
  const bool norm = job.xden != nullptr;
  const bool den = norm && job.xden != job.x;
  if (!norm) return launch_rows_k<T, 64, 64, false, false, 4, false, true>(p, job, job2, chunk, nchunks, 32, 32, st);
  if (!den) return launch_rows_k<T, 64, 64, true, false, 4, false, true>(p, job, job2, chunk, nchunks, 32, 32, st);
  return launch_rows_k<T, 64, 64, true, true, 4, false, true>(p, job, job2, chunk, nchunks, 32, 32, st);
}

template <typename T, bool PAD>
static int run_rows_dims(const Prob& p, const RowsJob& job, const RowsJob* job2, int dr, int dc,
                         hipStream_t st) {
  const int DR = tiled_dim(dr), DC = tiled_dim(dc);
  if (DR == 64 && DC == 64) return launch_rows<T, 64, 64, PAD>(p, job, job2, dr, dc, st);
  if (DR == 64) return launch_rows<T, 64, 128, PAD>(p, job, job2, dr, dc, st);
  if (DC == 64) return launch_rows<T, 128, 64, PAD>(p, job, job2, dr, dc, st);
  return launch_rows<T, 128, 128, PAD>(p, job, job2, dr, dc, st);
}

template <typename T>
static int run_rows(const Prob& p, const RowsJob& job, const RowsJob* job2, int dr, int dc,
                    hipStream_t st) {
  if (pair_mode(p, kF16) && job.pnchunks == 0) return launch_rows_pair<T>(p, job, job2, st);
  if (padded(p)) return run_rows_dims<T, true>(p, job, job2, dr, dc, st);
  return run_rows_dims<T, false>(p, job, job2, dr, dc, st);
}

// Packed batches, which kernels keep the workgroups of a sequence on one XCD (packed_item):
// bit 0 the state kernels, bit 1 the row-parallel kernels, bit 2 backward pass A.  The
// row-parallel kernels gain (their stores come in 128-byte pieces a token row apart, and the
// pieces of the other heads are then written at about the same time: forward output 89 -> 82 us,
// pass B 152 -> 145 us at 64 sequences, H=16, D=64; 3-7 % of forward and backward from 16 to
// 256 sequences); the reductions lose a little of the longest-first balance and gain nothing,
// and so do the row-parallel kernels with 128-wide tiles (one or two workgroups per CU, several
// rounds of them).
static bool small_tiles(int DR, int DC) { return tiled_dim(DR) == 64 && tiled_dim(DC) == 64; }
static Prob xcd_ordered(const Prob& p, int kernel_bit) {
  static const int mask = tuning_knob("FBLA_XCD_ORDER", 2, true);
  Prob r = p;
  if (p.cu && (mask & kernel_bit)) r.flags |= kXcdOrder;
  return r;
}

// Dense tensors, 16-bit heads tiled 64 x 64 (not the two-tokens-per-row mode): which kernels let
// the workgroups of a head take interleaved token steps (bit 0 the state kernel, bit 1 the
// row-parallel kernels, bit 2 backward pass A).
static int interleave_mask() {
  static const int mask = tuning_knob("FBLA_ILEAVE", 7, true);
  return mask;
}
bool interleaved(const Prob& p, int dtype, int kernel_bit) {
  return (interleave_mask() & kernel_bit) && !p.cu && dtype != kF32 && small_tiles(p.DK, p.DV) &&
         !pair_mode(p, dtype);
}
// Tokens per partial as the reduction sees them: workgroup c of an interleaved walk has work
// when c * granule < len.
int partial_chunk(const Prob& p, int dtype, int kernel_bit, int chunk) {
  return interleaved(p, dtype, kernel_bit) ? (kernel_bit == 1 ? 64 : 128) : chunk;
}
Prob with_interleave(const Prob& p, int dtype, int kernel_bit) {
  Prob r = p;
  if (interleaved(p, dtype, kernel_bit)) r.flags |= kInterleave;
  return r;
}

void state(const Prob& p_, int dtype, const void* kn, const void* v, const void* kd, float* partial,
           int chunk, int nchunks, hipStream_t st, float* fin_mat, float* fin_vec) {
  const Prob p = xcd_ordered(p_, 1);
  const BlockStats none{nullptr, nullptr, 0};
  if (dtype == kF32)
    return mfma32::state(p, (const float*)kn, (const float*)v, (const float*)kd, partial, nullptr, 0, chunk,
                         nchunks, st, fin_mat, fin_vec);
  if (dtype == kF16) run_state<_Float16>(p, kn, v, kd, partial, nullptr, 0, fin_mat, fin_vec, chunk, nchunks, none, st);
  else run_state<__bf16>(p, kn, v, kd, partial, nullptr, 0, fin_mat, fin_vec, chunk, nchunks, none, st);
}

void state_with_block_stats(const Prob& p, int dtype, const void* k, const void* v, float* partial,
                            int chunk, int nchunks, float* kc, float* vc, int NT, hipStream_t st) {
  const BlockStats bs{kc, vc, NT};
  if (dtype == kF16) run_state<_Float16>(p, k, v, k, partial, nullptr, 0, nullptr, nullptr, chunk, nchunks, bs, st);
  else run_state<__bf16>(p, k, v, k, partial, nullptr, 0, nullptr, nullptr, chunk, nchunks, bs, st);
}

void scaled_state(const Prob& p, int dtype, const void* qn, const void* qd, const void* dout,
                  const float* tokscal, int64_t total_rows, float* partial, int chunk, int nchunks,
                  hipStream_t st, float* fin_mat, float* fin_vec) {
  const BlockStats none{nullptr, nullptr, 0};
  if (dtype == kF32)
    return mfma32::state(p, (const float*)qn, (const float*)dout, (const float*)qd, partial, tokscal,
                         total_rows, chunk, nchunks, st, fin_mat, fin_vec);
  if (dtype == kF16)
    run_state<_Float16>(p, qn, dout, qd, partial, tokscal, total_rows, fin_mat, fin_vec, chunk, nchunks, none, st);
  else
    run_state<__bf16>(p, qn, dout, qd, partial, tokscal, total_rows, fin_mat, fin_vec, chunk, nchunks, none, st);
}

// (not for batches whose longest sequence is split into many chunks: all of them on one XCD would
// leave the other seven to the short sequences - one sequence of 65536 tokens among 63 of 256,
// H16-D64: forward output 286 -> 70 us, pass B 552 -> 120 us)
static bool xcd_order_rows(const Prob& p, int DR, int DC) {
  return small_tiles(DR, DC) && cdiv64(p.L, rows_chunk(p, DR, DC)) <= 4;
}

int rows(const Prob& p_, int dtype, const RowsJob& job, int DR, int DC, hipStream_t st) {
  const Prob p = xcd_order_rows(p_, DR, DC) ? xcd_ordered(p_, 2) : p_;
  if (dtype == kF32) return mfma32::rows(p, job, nullptr, DR, DC, st);
  if (dtype == kF16) return run_rows<_Float16>(p, job, nullptr, DR, DC, st);
  return run_rows<__bf16>(p, job, nullptr, DR, DC, st);
}

// two jobs of the same shape and normalisation mode in one launch
int rows2(const Prob& p_, int dtype, const RowsJob& job0, const RowsJob& job1, int DR, int DC,
          hipStream_t st) {
  const Prob p = xcd_order_rows(p_, DR, DC) ? xcd_ordered(p_, 2) : p_;
  if (dtype == kF32) return mfma32::rows(p, job0, &job1, DR, DC, st);
  if (dtype == kF16) return run_rows<_Float16>(p, job0, &job1, DR, DC, st);
  return run_rows<__bf16>(p, job0, &job1, DR, DC, st);
}

template <typename T, int DK, int DV, bool NORM, bool DEN, bool FUSED, bool PAD, bool PAIR = false, bool GATE = false,
          bool FMAP = false>
static int launch_bwd_a(const Prob& p, const T* qn, const T* qd, const T* dout, const float* S,
                        const float* km, T* dqn, T* dqd, float* partial, float* tokscal,
                        int64_t total_rows, float* fm, float* fv, int chunk, int nchunks,
                        hipStream_t st) {
  // dO / z enters the dS product as hi + lo for bf16; for fp16 (11 significant bits, and the
  // rounding errors of the tokens average out in the sum) the hi part alone: the gradients'
  // error against float64 moves from 3.6e-4 to 4.7e-4 of their largest element, the kernel
  // is 4 % faster.  The reference rounds this operand to the input type in both cases
  // (linear_attn/fused.py:238-242).
  constexpr bool LO = !std::is_same<T, _Float16>::value;
  using LY = BwdALayout<DK, DV, NORM, DEN, FUSED, LO>;
  static_assert(!FUSED || LY::kTotal - LY::kOpnd >=
                              (int)sizeof(float) * 64 * ((DK / 32) * (DV / 32) * 16 + DK / 32),
                "reduction buffer must fit in the tile area");
  static_assert(LY::kTotal <= 160 * 1024, "LDS budget of one workgroup");
  auto kernel = bwd_a_kernel<T, DK, DV, NORM, DEN, FUSED, LO, PAD, PAIR, GATE, FMAP>;
  static thread_local bool configured = false;  // per instantiation
  int rc = reserve_lds(kernel, LY::kTotal, configured);
  if (rc != kOk) return rc;
  const unsigned grid = (unsigned)((int64_t)p.N * p.H * nchunks);
  kernel<<<dim3(grid), dim3(kThreads), LY::kTotal, st>>>(p, qn, qd, dout, S, km, dqn, dqd, partial,
                                                         tokscal, total_rows, fm, fv, chunk, nchunks);
  return kOk;
}

template <typename T, bool NORM, bool PAD>
static int launch_bwd_a128(const Prob& p, const T* q, const T* dout, const float* S, const float* km, T* dq,
                           float* partial, float* fm, float* fv, int chunk, int nchunks, hipStream_t st) {
  using LY = BwdA128Layout;
  auto kernel = bwd_a128_kernel<T, NORM, PAD>;
  static thread_local bool configured = false;  // per instantiation
  int rc = reserve_lds(kernel, LY::kTotal, configured);
  if (rc != kOk) return rc;
  const unsigned grid = (unsigned)((int64_t)p.N * p.H * nchunks);
  kernel<<<dim3(grid), dim3(256), LY::kTotal, st>>>(p, q, dout, S, km, dq, partial, fm, fv, chunk, nchunks);
  return kOk;
}

template <typename T, bool PAD, bool PAIR = false>
static int run_bwd_a_pad(const Prob& p, const void* qn, const void* qd, const void* dout, const float* S,
                         const float* km, void* dqn, void* dqd, float* partial, float* fm, float* fv,
                         int chunk, int nchunks, hipStream_t st) {
  const T *a = (const T*)qn, *b = (const T*)qd, *c = (const T*)dout;
  T *x = (T*)dqn, *y = (T*)dqd;
  if constexpr (!PAIR) {
    if (tiled_dim(p.DK) == 128 || tiled_dim(p.DV) == 128) {
      if (!(p.flags & kNormalize))
        return launch_bwd_a128<T, false, PAD>(p, a, c, S, km, x, partial, fm, fv, chunk, nchunks, st);
      return launch_bwd_a128<T, true, PAD>(p, a, c, S, km, x, partial, fm, fv, chunk, nchunks, st);
    }
  }
  if constexpr (!PAD && !PAIR) {
    if (p.flags & kElu1Grad) {  // (the plan has checked: plain operator, 64 x 64)
      if (p.flags & kElu1) {  // q before the map
        if (!(p.flags & kNormalize))
          return launch_bwd_a<T, 64, 64, false, false, true, false, false, true, true>(p, a, b, c, S, km, x, y, partial, nullptr, 0, fm, fv, chunk, nchunks, st);
        return launch_bwd_a<T, 64, 64, true, false, true, false, false, true, true>(p, a, b, c, S, km, x, y, partial, nullptr, 0, fm, fv, chunk, nchunks, st);
      }
      if (!(p.flags & kNormalize))
        return launch_bwd_a<T, 64, 64, false, false, true, false, false, true>(p, a, b, c, S, km, x, y, partial, nullptr, 0, fm, fv, chunk, nchunks, st);
      return launch_bwd_a<T, 64, 64, true, false, true, false, false, true>(p, a, b, c, S, km, x, y, partial, nullptr, 0, fm, fv, chunk, nchunks, st);
    }
  }
  if (!(p.flags & kNormalize))
    return launch_bwd_a<T, 64, 64, false, false, true, PAD, PAIR>(p, a, b, c, S, km, x, y, partial, nullptr, 0, fm, fv, chunk, nchunks, st);
  if (p.flags & kDecoupled)
    return launch_bwd_a<T, 64, 64, true, true, true, PAD, PAIR>(p, a, b, c, S, km, x, y, partial, nullptr, 0, fm, fv, chunk, nchunks, st);
  return launch_bwd_a<T, 64, 64, true, false, true, PAD, PAIR>(p, a, b, c, S, km, x, y, partial, nullptr, 0, fm, fv, chunk, nchunks, st);
}

template <typename T>
static int run_bwd_a(const Prob& p, const void* qn, const void* qd, const void* dout, const float* S,
                     const float* km, void* dqn, void* dqd, float* partial, float* fm, float* fv,
                     int chunk, int nchunks, hipStream_t st) {
  // pair mode: the chunk (a multiple of 128 tokens) becomes a count of row pairs
  if (pair_mode(p, kF16))
    return run_bwd_a_pad<T, false, true>(p, qn, qd, dout, S, km, dqn, dqd, partial, fm, fv, chunk / 2, nchunks, st);
  if (padded(p) || tiled_dim(p.DK) != tiled_dim(p.DV)) return run_bwd_a_pad<T, true>(p, qn, qd, dout, S, km, dqn, dqd, partial, fm, fv, chunk, nchunks, st);
  return run_bwd_a_pad<T, false>(p, qn, qd, dout, S, km, dqn, dqd, partial, fm, fv, chunk, nchunks, st);
}

int bwd_a(const Prob& p_, int dtype, const void* qn, const void* qd, const void* dout, const float* S,
          const float* km, void* dqn, void* dqd, float* partial, int chunk, int nchunks,
          hipStream_t st, float* fin_mat, float* fin_vec) {
  const Prob p = xcd_ordered(p_, 4);
  if (dtype == kF16)
    return run_bwd_a<_Float16>(p, qn, qd, dout, S, km, dqn, dqd, partial, fin_mat, fin_vec, chunk, nchunks, st);
  return run_bwd_a<__bf16>(p, qn, qd, dout, S, km, dqn, dqd, partial, fin_mat, fin_vec, chunk, nchunks, st);
}

template <typename T, int DK, int DV, bool PAD>
static int launch_bwd_tokens(const Prob& p, const void* qn, const void* qd, const void* dout, const float* S,
                             const float* km, void* dqn, void* dqd, float* tokscal, int64_t total_rows,
                             int chunk, int nchunks, hipStream_t st) {
  const T *a = (const T*)qn, *b = (const T*)qd, *c = (const T*)dout;
  if (p.flags & kDecoupled)  // z from the plain q rows, dq = dz km next to dq_rope
    return launch_bwd_a<T, DK, DV, true, true, false, PAD>(p, a, b, c, S, km, (T*)dqn, (T*)dqd, nullptr, tokscal,
                                                           total_rows, nullptr, nullptr, chunk, nchunks, st);
  if (p.flags & kNormalize)
    return launch_bwd_a<T, DK, DV, true, false, false, PAD>(p, a, a, c, S, km, (T*)dqn, nullptr, nullptr,
                                                            tokscal, total_rows, nullptr, nullptr, chunk,
                                                            nchunks, st);
  return launch_bwd_a<T, DK, DV, false, false, false, PAD>(p, a, a, c, S, km, (T*)dqn, nullptr, nullptr,
                                                           tokscal, total_rows, nullptr, nullptr, chunk,
                                                           nchunks, st);
}

template <typename T, bool PAD>
static int run_bwd_tokens_dims(const Prob& p, const void* qn, const void* qd, const void* dout, const float* S,
                               const float* km, void* dqn, void* dqd, float* tokscal, int64_t total_rows,
                               int chunk, int nchunks, hipStream_t st) {
  const int DK = tiled_dim(p.DK), DV = tiled_dim(p.DV);
  if (DK == 64 && DV == 128)
    return launch_bwd_tokens<T, 64, 128, PAD>(p, qn, qd, dout, S, km, dqn, dqd, tokscal, total_rows, chunk, nchunks, st);
  if (DK == 128 && DV == 64)
    return launch_bwd_tokens<T, 128, 64, PAD>(p, qn, qd, dout, S, km, dqn, dqd, tokscal, total_rows, chunk, nchunks, st);
  if (DK == 128 && DV == 128 && (p.flags & kDecoupled))  // the plain operator has the fused 128 x 128 pass A
    return launch_bwd_tokens<T, 128, 128, PAD>(p, qn, qd, dout, S, km, dqn, dqd, tokscal, total_rows, chunk, nchunks, st);
  set_error("the token view alone exists for heads tiled 64 x 128, 128 x 64 and (decoupled) 128 x 128");
  return kErrUnsupported;
}

template <typename T>
static int run_bwd_tokens(const Prob& p, const void* qn, const void* qd, const void* dout, const float* S,
                          const float* km, void* dqn, void* dqd, float* tokscal, int64_t total_rows,
                          hipStream_t st) {
  const int big = (tiled_dim(p.DK) == 128) + (tiled_dim(p.DV) == 128);
  const int chunk = chunk_for(p, big == 2 ? 1 : 2, 1, 512, 128, false);
  const int nchunks = (int)cdiv64(p.L, chunk);
  if (padded(p))
    return run_bwd_tokens_dims<T, true>(p, qn, qd, dout, S, km, dqn, dqd, tokscal, total_rows, chunk, nchunks, st);
  return run_bwd_tokens_dims<T, false>(p, qn, qd, dout, S, km, dqn, dqd, tokscal, total_rows, chunk, nchunks, st);
}

// token view of the backward alone: dq and the per-row scalars 1/z_t, dz_t
int bwd_tokens(const Prob& p, int dtype, const void* qn, const void* qd, const void* dout, const float* S,
               const float* km, void* dqn, void* dqd, float* tokscal, int64_t total_rows, hipStream_t st) {
  if (dtype == kF32)
    return mfma32::bwd_tokens(p, (const float*)qn, (const float*)qd, (const float*)dout, S, km, (float*)dqn,
                              (float*)dqd, tokscal, total_rows, st);
  if (dtype == kF16) return run_bwd_tokens<_Float16>(p, qn, qd, dout, S, km, dqn, dqd, tokscal, total_rows, st);
  return run_bwd_tokens<__bf16>(p, qn, qd, dout, S, km, dqn, dqd, tokscal, total_rows, st);
}

}  // namespace mfma
}  // namespace fbla
