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
      a0 += to_f32(src[(int64_t)t * D + d]);
      a1 += to_f32(src[(int64_t)(t + 1) * D + d]);
      a2 += to_f32(src[(int64_t)(t + 2) * D + d]);
      a3 += to_f32(src[(int64_t)(t + 3) * D + d]);
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
    float* __restrict__ kc, float* __restrict__ vc, int64_t BH, int Tn, int NT, int chunk) {
  constexpr int CH = D / 8, RPI = 64 / CH;  // chunks per row, rows per wave instruction
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int64_t item = (int64_t)blockIdx.x * 4 + wave;
  if (item >= BH * NT * 3) return;
  const int which = (int)(item % 3);
  const int64_t bc = item / 3;
  const int c = (int)(bc % NT);
  const int64_t bh = bc / NT;
  const T* src = (which == 0 ? q : which == 1 ? k : v) + (bh * Tn + (int64_t)c * chunk) * D;
  float* dst = (which == 0 ? qc : which == 1 ? kc : vc) + bc * D;
  const int n = min(chunk, Tn - c * chunk);
  const int ch = lane % CH, r0 = lane / CH;
  float acc[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) acc[i] = 0.f;
  for (int base = 0; base < n; base += 4 * RPI) {
    u32x4s w[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int row = base + u * RPI + r0;
      w[u] = row < n ? *reinterpret_cast<const u32x4s*>(src + (int64_t)row * D + ch * 8)
                     : u32x4s{0u, 0u, 0u, 0u};
    }
#pragma unroll
    for (int u = 0; u < 4; ++u)
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
// statistics go through LDS in slabs of 64 chunks (coalesced loads, every value is
// then used 16 times from LDS); the chunk order of the sum is fixed.
constexpr int kHTile = 32, kHSlab = 64;
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
    for (int i = threadIdx.x; i < kHSlab * kHTile; i += kThreads) {
      const int c = i / kHTile, d = i % kHTile;
      ks[c][d] = (c < nc && dk0 + d < K) ? kch[(int64_t)(cb + c) * K + dk0 + d] : 0.f;
      vs[c][d] = (c < nc && dv0 + d < V) ? vch[(int64_t)(cb + c) * V + dv0 + d] : 0.f;
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
  const float corr[2][2] = {{c00, c01}, {c10, c11}};
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int dk = dk0 + 2 * ty + i, dv = dv0 + tx + 16 * j;
      if (dk >= K || dv >= V) continue;
      const int e = dk * V + dv;
      float a = 0.f;
      for (int pidx = 0; pidx < nparts; ++pidx) a += partial[(bh * nparts + pidx) * stride + e];
      h[bh * E + e] = a - corr[i][j];
    }
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

// ===========================================================================
// attention kernel
// ===========================================================================
// One workgroup (4 waves) per (head, 64-query block); each wave owns 16 queries.
// MFMA: v_mfma_f32_16x16x32_{f16,bf16} (A lane l: m=l%16, k=8*(l/16)+i; B lane l:
// n=l%16, k=8*(l/16)+i; C lane l: n=l%16, rows 4*(l/16)+r).  Scores are computed
// transposed, S^T = K Q^T, so that a lane holds 16 keys of ONE query: the row
// maximum needs two shuffles, and exp(S^T) packed to 16 bits is directly the B
// operand of O^T += V^T P^T (the key order of that contraction is chosen to match).
// V^T operands come from LDS with the dword + v_perm transposition.
//
//   phase 1  exact softmax attention over the NS selected 64-key blocks
//   phase 2  the unselected blocks, each represented by its mean key (weight n_c in
//            the denominator) and its value sum; means/sums are hi+lo 16-bit pairs
//   phase 3  first-order term: acc += (q H) * (G/T) * scale, q H precomputed per token
//   o = acc / (l + G)
// Unlike the Triton kernel (kernel.py:263-276) the running G is rescaled together
// with acc and l whenever the running maximum grows.
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

template <typename T> struct Mma16;
template <> struct Mma16<_Float16> {
  static __device__ __forceinline__ f32x4 run(u32x4 a, u32x4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a),
                                                  __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
};
template <> struct Mma16<__bf16> {
  static __device__ __forceinline__ f32x4 run(u32x4 a, u32x4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a),
                                                   __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
};
template <typename T> __device__ __forceinline__ uint32_t pack_pair(float a, float b) {
  return (uint32_t)__builtin_bit_cast(uint16_t, (T)a) |
         ((uint32_t)__builtin_bit_cast(uint16_t, (T)b) << 16);
}
template <typename T> __device__ __forceinline__ float unpack_lo(uint32_t w) {
  return (float)__builtin_bit_cast(T, (uint16_t)(w & 0xffffu));
}
template <typename T> __device__ __forceinline__ float unpack_hi(uint32_t w) {
  return (float)__builtin_bit_cast(T, (uint16_t)(w >> 16));
}

struct AttnArgs {
  const void *q, *k, *v;         // [BH, T, K], [BH, T, K], [BH, T, V]
  const void *kc_hi, *kc_lo;     // [BH, NTp, K] 16-bit: chunk mean keys, hi + lo
  const void *vc_hi, *vc_lo;     // [BH, NTp, V] 16-bit: chunk value sums, hi + lo
  const void* r;                 // [BH, T, V] 16-bit: q H per token
  const int32_t* indices;        // [BH, NT, NS] selected key blocks per query block
  void* o;                       // [BH, T, V]
  int T, NT, NTp, NS;
  float scale;
};

template <int K, int V> struct AttnLayout {
  static constexpr int kKT = 64 * K * 2, kVT = 64 * V * 2;  // one 64-row tile
  static constexpr int kSet = kKT + kVT;
  static constexpr int kSel = 2 * kSet;
  static constexpr int kTotalNoSel = 2 * kSet;
};

template <typename T, int K, int V>
__global__ __launch_bounds__(kThreads) void attention_kernel(AttnArgs a) {
  using LY = AttnLayout<K, V>;
  constexpr int KCH = K / 8, VCH = V / 8;        // 16-byte chunks per row
  constexpr int KST = K / 32;                    // k-steps of the score product
  constexpr int DG = V / 32;                     // 32-wide value column groups
  constexpr int KLD = 64 * KCH / kThreads, VLD = 64 * VCH / kThreads;  // chunks per thread per tile
  constexpr float kNegInf = -__builtin_huge_valf();
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  unsigned char* sel = smem + LY::kSel;

  const int tq = blockIdx.x % a.NT;
  const int64_t bh = blockIdx.x / a.NT;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int nq = lane & 15, kb = lane >> 4;
  const int qtok = tq * 64 + wave * 16 + nq;  // this lane's query token
  const float sm_scale = a.scale * 1.44269504f;

  const T* qb = (const T*)a.q + bh * a.T * K;
  const T* kbase = (const T*)a.k + bh * a.T * K;
  const T* vbase = (const T*)a.v + bh * a.T * V;

  // selected-block bitmap
  for (int i = tid; i < a.NTp; i += kThreads) sel[i] = 0;
  __syncthreads();
  const int32_t* idx = a.indices + (bh * a.NT + tq) * a.NS;
  for (int i = tid; i < a.NS; i += kThreads) {
    const int b = idx[i];
    if (b >= 0 && b < a.NT) sel[b] = 1;
  }

  // Q^T operand: k-step s covers d = 32s + 8kb + i
  u32x4 qop[KST];
#pragma unroll
  for (int s = 0; s < KST; ++s)
    qop[s] = qtok < a.T ? *reinterpret_cast<const u32x4*>(qb + (int64_t)qtok * K + 32 * s + 8 * kb)
                        : u32x4{0u, 0u, 0u, 0u};

  // tile swizzles: K rows are read 16 B per lane down a column of 16 rows; V rows are
  // read one dword per lane, four rows (one per kb) at a time
  auto kswz = [](int row, int ch) { return row * (K * 2) + ((ch ^ (row & 7)) << 4); };
  auto vswz_chunk = [](int row, int ch) { return row * (V * 2) + ((ch ^ (((row >> 2) & 1) << 2)) << 4); };
  auto vswz_dword = [](int row, int dw) { return row * (V * 2) + ((dw ^ (((row >> 2) & 1) << 4)) << 2); };

  auto load_tile_k = [&](u32x4(&dst)[KLD], const T* src, int row0, int nrows) {
#pragma unroll
    for (int j = 0; j < KLD; ++j) {
      const int qq = tid + kThreads * j, row = qq / KCH, ch = qq % KCH;
      dst[j] = row < nrows ? *reinterpret_cast<const u32x4*>(src + (int64_t)(row0 + row) * K + ch * 8)
                           : u32x4{0u, 0u, 0u, 0u};
    }
  };
  auto load_tile_v = [&](u32x4(&dst)[VLD], const T* src, int row0, int nrows) {
#pragma unroll
    for (int j = 0; j < VLD; ++j) {
      const int qq = tid + kThreads * j, row = qq / VCH, ch = qq % VCH;
      dst[j] = row < nrows ? *reinterpret_cast<const u32x4*>(src + (int64_t)(row0 + row) * V + ch * 8)
                           : u32x4{0u, 0u, 0u, 0u};
    }
  };
  auto store_tile_k = [&](const u32x4(&src)[KLD], unsigned char* tile) {
#pragma unroll
    for (int j = 0; j < KLD; ++j) {
      const int qq = tid + kThreads * j;
      *reinterpret_cast<u32x4*>(tile + kswz(qq / KCH, qq % KCH)) = src[j];
    }
  };
  auto store_tile_v = [&](const u32x4(&src)[VLD], unsigned char* tile) {
#pragma unroll
    for (int j = 0; j < VLD; ++j) {
      const int qq = tid + kThreads * j;
      *reinterpret_cast<u32x4*>(tile + vswz_chunk(qq / VCH, qq % VCH)) = src[j];
    }
  };

  // per-lane LDS offsets of the operand reads (everything else is a compile-time constant)
  int koff[KST], voff[DG];
#pragma unroll
  for (int s = 0; s < KST; ++s) koff[s] = kswz(nq, 4 * s + kb);
#pragma unroll
  for (int dg = 0; dg < DG; ++dg) voff[dg] = vswz_dword(4 * kb, 16 * dg + nq);

  float m_i = kNegInf, l_p = 0.f, g_p = 0.f;  // running max; per-lane partial sums
  f32x4 acc[DG][2];
#pragma unroll
  for (int dg = 0; dg < DG; ++dg)
#pragma unroll
    for (int par = 0; par < 2; ++par) acc[dg][par] = f32x4{0.f, 0.f, 0.f, 0.f};

  // One 64-key block: scores against NKT key tiles (summed), masked, online softmax,
  // then acc += P (V tile 0 [+ V tile 1]).  valid(key) / weight(key) describe the block.
  auto attend = [&](const unsigned char* kt0, const unsigned char* kt1, const unsigned char* vt0,
                    const unsigned char* vt1, auto valid, auto weight, bool weighted, bool all_valid) {
    f32x4 st[4];
#pragma unroll
    for (int jb = 0; jb < 4; ++jb) {
      st[jb] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s = 0; s < KST; ++s) {
        // row 16jb + nq: same swizzle as row nq (16jb is a multiple of 8)
        const u32x4 ak = *reinterpret_cast<const u32x4*>(kt0 + koff[s] + jb * (16 * K * 2));
        st[jb] = Mma16<T>::run(ak, qop[s], st[jb]);
        if (kt1) {
          const u32x4 al = *reinterpret_cast<const u32x4*>(kt1 + koff[s] + jb * (16 * K * 2));
          st[jb] = Mma16<T>::run(al, qop[s], st[jb]);
        }
      }
    }
    // this lane: keys 16jb + 4kb + r of query nq
    float mx = kNegInf;
#pragma unroll
    for (int jb = 0; jb < 4; ++jb)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float x = (all_valid || valid(16 * jb + 4 * kb + r)) ? st[jb][r] * sm_scale : kNegInf;
        st[jb][r] = x;
        mx = fmaxf(mx, x);
      }
    mx = fmaxf(mx, __shfl_xor(mx, 16));
    mx = fmaxf(mx, __shfl_xor(mx, 32));
    const float m_new = fmaxf(m_i, mx);
    const float m_safe = m_new == kNegInf ? 0.f : m_new;
    const float alpha = __builtin_amdgcn_exp2f(m_i - m_safe);
    m_i = m_new;
    float psum = 0.f, wsum = 0.f;
    uint32_t pw[8];
#pragma unroll
    for (int jb = 0; jb < 4; ++jb) {
      float pv[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        pv[r] = __builtin_amdgcn_exp2f(st[jb][r] - m_safe);
        psum += pv[r];
        if (weighted) wsum = fmaf(pv[r], weight(16 * jb + 4 * kb + r), wsum);
      }
      pw[2 * jb] = pack_pair<T>(pv[0], pv[1]);
      pw[2 * jb + 1] = pack_pair<T>(pv[2], pv[3]);
    }
    if (weighted) {
      g_p = g_p * alpha + wsum;
      l_p = l_p * alpha;
    } else {
      l_p = l_p * alpha + psum;
      g_p = g_p * alpha;
    }
    if (__any(alpha != 1.f)) {  // the running maximum rarely moves after the first blocks
#pragma unroll
      for (int dg = 0; dg < DG; ++dg)
#pragma unroll
        for (int par = 0; par < 2; ++par) acc[dg][par] *= alpha;
    }
    // O^T += V^T P^T: k-step sp covers key sub-blocks 2sp, 2sp+1; slot i of lane kb is
    // key 32sp + 4kb + i (i < 4) or 32sp + 16 + 4kb + (i - 4)
#pragma unroll
    for (int sp = 0; sp < 2; ++sp) {
      const u32x4 bp = u32x4{pw[4 * sp], pw[4 * sp + 1], pw[4 * sp + 2], pw[4 * sp + 3]};
#pragma unroll
      for (int dg = 0; dg < DG; ++dg) {
#pragma unroll
        for (int tile = 0; tile < 2; ++tile) {
          const unsigned char* vt = tile == 0 ? vt0 : vt1;
          if (!vt) continue;
          uint32_t w[8];
#pragma unroll
          for (int i = 0; i < 8; ++i) {
            // row 32sp + 16(i/4) + 4kb + i%4: the swizzle bit (row/4)%2 equals kb%2 as in row 4kb
            w[i] = *reinterpret_cast<const uint32_t*>(vt + voff[dg] +
                                                      (32 * sp + 16 * (i >> 2) + (i & 3)) * (V * 2));
          }
          u32x4 ae, ao;
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            ae[i] = __builtin_amdgcn_perm(w[2 * i + 1], w[2 * i], 0x05040100u);
            ao[i] = __builtin_amdgcn_perm(w[2 * i + 1], w[2 * i], 0x07060302u);
          }
          acc[dg][0] = Mma16<T>::run(ae, bp, acc[dg][0]);
          acc[dg][1] = Mma16<T>::run(ao, bp, acc[dg][1]);
        }
      }
    }
  };

  // ---- phase 1: selected blocks, K/V tiles double-buffered ----
  u32x4 rk[KLD], rv[VLD];
  // rows of block b that exist (0 for an index outside [0, NT): the block is skipped)
  auto block_rows = [&](int b) { return b >= 0 && b < a.NT ? min(64, a.T - b * 64) : 0; };
  {
    const int b0 = idx[0], n0 = block_rows(b0);
    load_tile_k(rk, kbase, n0 ? b0 * 64 : 0, n0);
    load_tile_v(rv, vbase, n0 ? b0 * 64 : 0, n0);
    store_tile_k(rk, smem);
    store_tile_v(rv, smem + LY::kKT);
  }
  __syncthreads();
  for (int i = 0; i < a.NS; ++i) {
    const int blk = idx[i];
    unsigned char* cur = smem + (i & 1) * LY::kSet;
    unsigned char* nxt = smem + ((i + 1) & 1) * LY::kSet;
    const bool more = i + 1 < a.NS;
    if (more) {
      const int bn = idx[i + 1], nn = block_rows(bn);
      load_tile_k(rk, kbase, nn ? bn * 64 : 0, nn);
      load_tile_v(rv, vbase, nn ? bn * 64 : 0, nn);
    }
    const int nrows = block_rows(blk);
    attend(cur, nullptr, cur + LY::kKT, nullptr, [&](int key) { return key < nrows; },
           [](int) { return 0.f; }, false, nrows == 64);
    if (more) {
      store_tile_k(rk, nxt);
      store_tile_v(rv, nxt + LY::kKT);
    }
    __syncthreads();
  }

  // ---- phase 2: unselected blocks through their means / sums ----
  const int last_len = a.T - (a.NT - 1) * 64;
  for (int grp = 0; grp * 64 < a.NT; ++grp) {
    const int64_t row0 = bh * a.NTp + grp * 64;
    // four tiles: kc hi | vc hi | kc lo | vc lo
    {
      const T* src = (const T*)a.kc_hi + row0 * K;
      load_tile_k(rk, src, 0, 64);
      store_tile_k(rk, smem);
      src = (const T*)a.kc_lo + row0 * K;
      load_tile_k(rk, src, 0, 64);
      store_tile_k(rk, smem + LY::kSet);
      const T* vsrc = (const T*)a.vc_hi + row0 * V;
      load_tile_v(rv, vsrc, 0, 64);
      store_tile_v(rv, smem + LY::kKT);
      vsrc = (const T*)a.vc_lo + row0 * V;
      load_tile_v(rv, vsrc, 0, 64);
      store_tile_v(rv, smem + LY::kSet + LY::kKT);
    }
    __syncthreads();
    const int c0 = grp * 64;
    attend(smem, smem + LY::kSet, smem + LY::kKT, smem + LY::kSet + LY::kKT,
           [&](int key) { return c0 + key < a.NT && !sel[c0 + key]; },
           [&](int key) { return c0 + key == a.NT - 1 ? (float)last_len : 64.f; }, true, false);
    __syncthreads();
  }

  // ---- phase 3 and output ----
  float L = l_p, G = g_p;
  L += __shfl_xor(L, 16);
  L += __shfl_xor(L, 32);
  G += __shfl_xor(G, 16);
  G += __shfl_xor(G, 32);
  {
    const T* rsrc = (const T*)a.r + (bh * a.T + (int64_t)tq * 64) * V;
    load_tile_v(rv, rsrc, 0, a.T - tq * 64);
    store_tile_v(rv, smem + LY::kKT);
  }
  __syncthreads();
  const float corr = G / (float)a.T * a.scale;
  const float inv = 1.f / (L + G);
  unsigned char* rt = smem + LY::kKT;    // q H tile
  unsigned char* ot = smem + LY::kSet + LY::kKT;  // output tile
  const int qrow = wave * 16 + nq;
#pragma unroll
  for (int dg = 0; dg < DG; ++dg)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      // acc[dg][par][r] is value column 32dg + 2(4kb + r) + par: one dword per (dg, r)
      const int dw = 16 * dg + 4 * kb + r;
      const uint32_t rw = *reinterpret_cast<const uint32_t*>(rt + vswz_dword(qrow, dw));
      const float o0 = (acc[dg][0][r] + unpack_lo<T>(rw) * corr) * inv;
      const float o1 = (acc[dg][1][r] + unpack_hi<T>(rw) * corr) * inv;
      *reinterpret_cast<uint32_t*>(ot + vswz_dword(qrow, dw)) = pack_pair<T>(o0, o1);
    }
  __syncthreads();
  T* ob = (T*)a.o + (bh * a.T + (int64_t)tq * 64) * V;
#pragma unroll
  for (int j = 0; j < VLD; ++j) {
    const int qq = tid + kThreads * j, row = qq / VCH, ch = qq % VCH;
    if (tq * 64 + row < a.T)
      *reinterpret_cast<u32x4*>(ob + (int64_t)row * V + ch * 8) =
          *reinterpret_cast<const u32x4*>(ot + vswz_chunk(row, ch));
  }
}

// kc (fp32 mean) / vc (fp32 sum) -> zero-padded 16-bit hi + lo arrays [BH, NTp, D]
template <typename T>
__global__ __launch_bounds__(kThreads) void split_hi_lo_kernel(const float* __restrict__ src,
                                                               T* __restrict__ hi, T* __restrict__ lo,
                                                               int64_t BH, int NT, int NTp, int D) {
  const int64_t total = BH * NTp * D;
  for (int64_t e = (int64_t)blockIdx.x * kThreads + threadIdx.x; e < total;
       e += (int64_t)gridDim.x * kThreads) {
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

static Prob dense_prob(int64_t BH, int64_t T, int K, int V) {
  Prob p;
  p.cu = nullptr;
  p.N = (int)BH;
  p.H = 1;
  p.L = (int)T;
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
  return mfma::supported(p, dtype) ? mfma::state_chunk(p) : generic::state_chunk(p);
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
                        int64_t BH, int Tn, int NT, int chunk, int K, int V, hipStream_t st) {
  const int64_t items = BH * NT * 3;
  if constexpr (sizeof(T) == 2) {
    const dim3 grid((unsigned)cdiv64(items, 4)), block(kThreads);
    if (K == 64 && V == 64) {
      chunk_sums16_kernel<T, 64><<<grid, block, 0, st>>>((const T*)q, (const T*)k, (const T*)v, qc, kc, vc, BH, Tn, NT, chunk);
      return;
    }
    if (K == 128 && V == 128) {
      chunk_sums16_kernel<T, 128><<<grid, block, 0, st>>>((const T*)q, (const T*)k, (const T*)v, qc, kc, vc, BH, Tn, NT, chunk);
      return;
    }
  }
  chunk_sums_kernel<T><<<dim3((unsigned)cdiv64(items, 4)), dim3(kThreads), 0, st>>>(
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
  if (dtype == kF16) launch_sums<_Float16>(q, k, v, qc, kc, vc, BH, (int)T, NT, chunk, K, V, st);
  else if (dtype == kBF16) launch_sums<__bf16>(q, k, v, qc, kc, vc, BH, (int)T, NT, chunk, K, V, st);
  else launch_sums<float>(q, k, v, qc, kc, vc, BH, (int)T, NT, chunk, K, V, st);
  if (mfma::supported(p, dtype)) mfma::state(p, dtype, k, v, k, partial, sc, nparts, st);
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
         block == 64;
}

static int64_t padded_chunks(int64_t T) { return cdiv64(cdiv64(T, 64), 64) * 64; }

// kc_hi | kc_lo | vc_hi | vc_lo | r
size_t attention_workspace_bytes(int64_t BH, int64_t T, int K, int V) {
  const int64_t NTp = padded_chunks(T);
  return 2 * align_up((size_t)BH * NTp * K * 2, 256) + 2 * align_up((size_t)BH * NTp * V * 2, 256) +
         align_up((size_t)BH * T * V * 2, 256);
}

template <typename T, int K, int V>
static int launch_attention(const AttnArgs& a, int64_t BH, hipStream_t st) {
  using LY = AttnLayout<K, V>;
  const int lds = LY::kSel + a.NTp;
  if (lds > 160 * 1024) {
    set_error("piecewise attention: %d key blocks need more LDS than a workgroup has", a.NT);
    return kErrUnsupported;
  }
  auto kernel = attention_kernel<T, K, V>;
  static thread_local int reserved = 0;
  if (lds > reserved) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, lds);
    if (e != hipSuccess) {
      set_error("piecewise attention: cannot reserve %d bytes of LDS: %s", lds, hipGetErrorString(e));
      return kErrLaunch;
    }
    reserved = lds;
  }
  kernel<<<dim3((unsigned)(BH * a.NT)), dim3(kThreads), lds, st>>>(a);
  return kOk;
}

template <typename T>
static int attention_t(const void* q, const void* k, const void* v, const float* kc, const float* vc,
                       const float* h, const int32_t* indices, void* o, void* workspace, int64_t BH,
                       int64_t Tn, int K, int V, int NS, float scale, int dtype, hipStream_t st) {
  const int NT = (int)cdiv64(Tn, 64);
  const int64_t NTp = padded_chunks(Tn);
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
  split_hi_lo_kernel<T><<<dim3(gk), dim3(kThreads), 0, st>>>(kc, kc_hi, kc_lo, BH, NT, (int)NTp, K);
  split_hi_lo_kernel<T><<<dim3(gv), dim3(kThreads), 0, st>>>(vc, vc_hi, vc_lo, BH, NT, (int)NTp, V);
  // r_t = q_t H: the row-parallel kernel with M = H
  const Prob p = dense_prob(BH, Tn, K, V);
  mfma::RowsJob job{q, nullptr, h, V, 1, nullptr, nullptr, r};
  int rc = mfma::rows(p, dtype, job, K, V, st);
  if (rc != kOk) return rc;
  AttnArgs a{q, k, v, kc_hi, kc_lo, vc_hi, vc_lo, r, indices, o, (int)Tn, NT, (int)NTp, NS, scale};
  if (K == 64 && V == 64) return launch_attention<T, 64, 64>(a, BH, st);
  if (K == 64) return launch_attention<T, 64, 128>(a, BH, st);
  if (V == 64) return launch_attention<T, 128, 64>(a, BH, st);
  return launch_attention<T, 128, 128>(a, BH, st);
}

int attention(const void* q, const void* k, const void* v, const float* kc, const float* vc,
              const float* h, const int32_t* indices, void* o, void* workspace, int64_t BH, int64_t T,
              int K, int V, int NS, float scale, int dtype, hipStream_t st) {
  if (dtype == kF16)
    return attention_t<_Float16>(q, k, v, kc, vc, h, indices, o, workspace, BH, T, K, V, NS, scale, dtype, st);
  return attention_t<__bf16>(q, k, v, kc, vc, h, indices, o, workspace, BH, T, K, V, NS, scale, dtype, st);
}

}  // namespace piecewise
}  // namespace fbla
