// MFMA kernels for fp32 inputs, heads tiled 64 x 64 (larger heads: fbla_mfma32w.hip): head dims that
// are multiples of 4 (16-byte row pieces) up to 64, smaller ones with zero padding (PAD variants: true row lengths in memory,
// missing features read as zero, outputs and state in their true shapes).  Dense and packed
// layouts, with or without the denominator, plain and decoupled (numerator from the rotary
// features, denominator from the plain ones).  v_mfma_f32_32x32x2_f32 computes in fp32 throughout, so
// there is no operand splitting here: A lane l holds A[m = l%32][k = l/32], B lane l
// holds B[k = l/32][n = l%32], C register r of lane l is C[8*(r/4) + 4*(l/32) + r%4][l%32].
// One instruction covers two values of the contraction index and takes 64 cycles:
// at 16 flop per byte these kernels keep the matrix unit about half busy at HBM speed.
//
//  state32_kernel   S_part = K^T V and sum_t k_t over a token chunk.  A lane owns one
//                   feature of the token rows 2s + kb: row loads are 128 contiguous
//                   bytes per half-wave and need no transposition at all.  SCALED: the
//                   feature view of the backward, v = dO scaled by 1/z_t per row and the
//                   vector part sum_t dz_t q_t.
//  rows32_kernel    out_t = (x_t M) * rowscale_t + addvec: forward output and both
//                   products of backward pass B.  TOKENS: the token view of backward
//                   pass A (x = dO, M = S^T; then q.g, z, dz, dq and the per-row scalars).
// The backward pass A is therefore two kernels (5 tensor passes), as for the 16-bit decoupled
// operator with a 128-wide side.
#include <stdlib.h>

#include "fbla_kernels.h"
#include "fbla_mfma_shared.h"

namespace fbla {
namespace mfma32 {

using mfma::f32x16;
using mfma::kLptMax;
using mfma::lpt_sequence;
using mfma::reduce_store_block;
using mfma::stream_load;
using mfma::stream_store;
using mfma::swz;
using mfma::wave_sync;

typedef float f32x4 __attribute__((ext_vector_type(4)));
// streaming hint per access class: 1 = state kernel loads, 2 = rows kernel tile loads,
// 4 = rows kernel stores
#ifndef FBLA_NT32
#define FBLA_NT32 7
#endif
typedef float f32x2 __attribute__((ext_vector_type(2)));

constexpr int kThreads = 256;
constexpr int kWaves = 4;
constexpr int D = 64;  // head dim of both operands

__device__ __forceinline__ f32x16 mma(float a, float b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
}

// ===========================================================================
// state kernel
// ===========================================================================
// Lane l = (f = l%32, kb = l/32).  A 16-token tile is eight k-steps; in k-step s the lane
// holds feature 32a + f of token 2s + kb for the key blocks a = 0, 1 and the value blocks
// b = 0, 1.  Four waves take interleaved tiles; two register buffers alternate.
template <bool SPLIT_KD, bool SCALED, bool PAD>
__global__ __launch_bounds__(kThreads, 2) void state32_kernel(
    Prob p, const float* __restrict__ kn, const float* __restrict__ v, const float* __restrict__ kd,
    float* __restrict__ partial, const float* __restrict__ tokscal, int64_t total_rows, float* fin_mat,
    float* fin_vec, int chunk, int nchunks) {
  __shared__ float red[64 * 66];
  __shared__ int lpt_lens[kLptMax + 1];
  const int dk = PAD ? p.DK : D, dv = PAD ? p.DV : D;  // row lengths in memory
  const int wg_nh = blockIdx.x / nchunks, c = blockIdx.x - wg_nh * nchunks;
  const int h = wg_nh % p.H;
  const int n = lpt_sequence(p, wg_nh / p.H, lpt_lens);
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

  const int g = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int f = lane & 31, kb = lane >> 5;
  // this lane's two key and two value features; one past the head dim is read from column 0
  // and replaced by zero
  bool kok[2], vok[2];
  int kcol[2], vcol[2];
#pragma unroll
  for (int a = 0; a < 2; ++a) {
    kok[a] = !PAD || f + 32 * a < dk;
    vok[a] = !PAD || f + 32 * a < dv;
    kcol[a] = kok[a] ? f + 32 * a : 0;
    vcol[a] = vok[a] ? f + 32 * a : 0;
  }

  f32x16 acc[2][2];
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.f;
  float ks[2] = {0.f, 0.f};

  struct Buf {
    float k[8][2], v[8][2];
    float d[SPLIT_KD ? 8 : 1][2];
    float rz[SCALED ? 8 : 1], dz[SCALED ? 8 : 1];
  };
  const uint32_t kstep = (uint32_t)(rstride * dk), vstep = (uint32_t)(rstride * dv);
  // A tile that would cross the end of the chunk is moved back so that it ends there; the
  // rows it shares with the previous tile are zeroed before use.
  auto fetch = [&](Buf& b, int tok) {
    const int tb = min(tok, t_end - 16);
    const int64_t row = row0 + (int64_t)tb * rstride;
    const float* kp = kn + row * dk;
    const float* vp = v + row * dv;
    const float* dp = kd + row * dk;
#pragma unroll
    for (int s = 0; s < 8; ++s) {
      const size_t kro = (size_t)(2 * s + kb) * kstep, vro = (size_t)(2 * s + kb) * vstep;
#pragma unroll
      for (int a = 0; a < 2; ++a) {
        const float kx = stream_load<(FBLA_NT32 & 1) != 0, float>(kp + kro + kcol[a]);
        const float vx = stream_load<(FBLA_NT32 & 1) != 0, float>(vp + vro + vcol[a]);
        b.k[s][a] = kok[a] ? kx : 0.f;
        b.v[s][a] = vok[a] ? vx : 0.f;
        if constexpr (SPLIT_KD) {
          const float dx = stream_load<(FBLA_NT32 & 1) != 0, float>(dp + kro + kcol[a]);
          b.d[s][a] = kok[a] ? dx : 0.f;
        }
      }
      if constexpr (SCALED) {
        const int64_t r = row + (int64_t)(2 * s + kb) * rstride;
        b.rz[s] = tokscal[r];
        b.dz[s] = tokscal[total_rows + r];
      }
    }
  };
  auto fetch_checked = [&](Buf& b, int tok) {  // chunk shorter than a tile
#pragma unroll
    for (int s = 0; s < 8; ++s) {
      const int t = tok + 2 * s + kb;
      const bool ok = t < t_end;
      const int64_t r = row0 + (int64_t)t * rstride;
#pragma unroll
      for (int a = 0; a < 2; ++a) {
        b.k[s][a] = ok && kok[a] ? kn[r * dk + kcol[a]] : 0.f;
        b.v[s][a] = ok && vok[a] ? v[r * dv + vcol[a]] : 0.f;
        if constexpr (SPLIT_KD) b.d[s][a] = ok && kok[a] ? kd[r * dk + kcol[a]] : 0.f;
      }
      if constexpr (SCALED) {
        b.rz[s] = ok ? tokscal[r] : 0.f;
        b.dz[s] = ok ? tokscal[total_rows + r] : 0.f;
      }
    }
  };
  auto compute = [&](Buf& b, int tok, bool checked) {
    if (!checked && tok + 16 > t_end) {
      const int lo = tok - (t_end - 16);  // rows below lo belong to the previous tile
#pragma unroll
      for (int s = 0; s < 8; ++s) {
        const bool keep = 2 * s + kb >= lo;
#pragma unroll
        for (int a = 0; a < 2; ++a) {
          b.k[s][a] = keep ? b.k[s][a] : 0.f;
          if constexpr (SPLIT_KD) b.d[s][a] = keep ? b.d[s][a] : 0.f;
        }
        if constexpr (SCALED) b.dz[s] = keep ? b.dz[s] : 0.f;
      }
    }
#pragma unroll
    for (int s = 0; s < 8; ++s) {
      float vv[2] = {b.v[s][0], b.v[s][1]};
      if constexpr (SCALED) {
        vv[0] *= b.rz[s];
        vv[1] *= b.rz[s];
      }
#pragma unroll
      for (int a = 0; a < 2; ++a) {
#pragma unroll
        for (int bb = 0; bb < 2; ++bb) acc[a][bb] = mma(b.k[s][a], vv[bb], acc[a][bb]);
        if constexpr (SCALED) ks[a] = fmaf(b.dz[s], SPLIT_KD ? b.d[s][a] : b.k[s][a], ks[a]);
        else ks[a] += SPLIT_KD ? b.d[s][a] : b.k[s][a];
      }
    }
  };
  int t0 = t_begin + 16 * g;
  if (t_end - t_begin < 16) {
    if (t0 < t_end) {
      Buf b0;
      fetch_checked(b0, t0);
      compute(b0, t0, true);
    }
  } else if (t0 < t_end) {
    Buf b0, b1;
    fetch(b0, t0);
    while (true) {
      fetch(b1, t0 + 16 * kWaves);
      compute(b0, t0, false);
      t0 += 16 * kWaves;
      if (t0 >= t_end) break;
      fetch(b0, t0 + 16 * kWaves);
      compute(b1, t0, false);
      t0 += 16 * kWaves;
      if (t0 >= t_end) break;
    }
  }

  float* mat = fin_mat ? fin_mat + (int64_t)nh * dk * dv
                       : partial + ((int64_t)nh * nchunks + c) * (dk * dv + dk);
  float* vec = fin_mat ? (fin_vec ? fin_vec + (int64_t)nh * dk : nullptr) : mat + dk * dv;
  const float mscale = fin_mat ? seq_scale(p, len) : 1.f;
  const float vscale = fin_mat ? 1.0f / (float)len : 1.f;
  reduce_store_block<4, false>(acc, ks, red, mat, dv, vec, mscale, vscale, g, lane, dk, dv);
}

// ===========================================================================
// rows kernel
// ===========================================================================
// C[m][n = token] = sum_k A[m][k] B[k][n] with A = the operand M (from LDS) and B = x.
// The contraction index of k-step s and half-wave kb is feature r(s, kb) = 4*(s/2) + 2*kb
// + s%2: a lane's B values of k-steps 2i, 2i+1 are then 8 contiguous bytes of the staged
// x tile, and the A values of four k-steps one 16-byte read.  Row m = 8g + 4kb' + j of
// block b is output feature sigma(b, m) = 32*kb' + 16*b + 4*g + j: after the MFMA a lane
// (token, kb') owns 32 consecutive output features.
//
// Operand fragments in LDS: frag[((b*8 + s/4)*64 + lane)*4 + s%4] = M[r(s,kb)][sigma(b,m)],
// lane = m + 32*kb.  M is read as mat[r*ld_r + c*ld_c] times mscale.
// The matrix in memory is dr x dc; rows and columns past that are zero in the operand.
__device__ __forceinline__ void build_operand32(float* frag, const float* __restrict__ mat, int ld_r,
                                                int ld_c, float mscale, int dr, int dc) {
  // a thread's elements are all requested before the first is stored (clamped addresses instead
  // of branches: a loop of guarded loads waits for every single one)
  constexpr int kPer = D * D / kThreads;
  float val[kPer];
  const bool c_fast = ld_c == 1;  // walk the matrix along its contiguous direction
#pragma unroll
  for (int i = 0; i < kPer; ++i) {
    const int e = threadIdx.x + i * kThreads;
    const int r = c_fast ? e / D : e % D, cc = c_fast ? e % D : e / D;
    const bool in = r < dr && cc < dc;
    val[i] = mat[in ? (int64_t)r * ld_r + (int64_t)cc * ld_c : 0];
    val[i] = in ? val[i] * mscale : 0.f;
  }
#pragma unroll
  for (int i = 0; i < kPer; ++i) {
    const int e = threadIdx.x + i * kThreads;
    const int r = c_fast ? e / D : e % D, cc = c_fast ? e % D : e / D;
    const int s = 2 * (r >> 2) + (r & 1), kb = (r >> 1) & 1;
    const int kbp = cc >> 5, b = (cc >> 4) & 1, gq = (cc >> 2) & 3, j = cc & 3;
    const int m = 8 * gq + 4 * kbp + j;
    frag[((b * 8 + (s >> 2)) * 64 + m + 32 * kb) * 4 + (s & 3)] = val[i];
  }
}

struct Rows32Job {
  const float* x;       // [rows, 64] B operand
  const float* xnum;    // TOKENS: the rows q~ of the numerator (q_rope when decoupled, else q)
  float* out2;          // TOKENS, decoupled: dq = dz km (out then holds dq~ = g / z)
  const float* xden;    // NORM: rows for the denominator (x itself unless decoupled); TOKENS: q
  const float* mat;     // operand M, element (r, c) at mat[nh*4096 + r*ld_r + c*ld_c]
  int ld_r, ld_c;
  const float* km;      // [NH, 64] mean key (NORM / TOKENS with the denominator)
  const float* addvec;  // [NH, 64] added (times add_scale) to every output row, or null
  float add_scale;
  float* out;           // [rows, 64]
  float* tokscal;       // TOKENS: [2][total rows]: 1/z_t, dz_t
  int64_t total_rows;
  int dr, dc;           // row lengths of x and out in memory (<= 64, multiples of 4)
};

struct Rows32Layout {
  static constexpr int kFrag = D * D * 4;        // 16 KiB
  static constexpr int kStage = 32 * D * 4;      // one 32-token tile, 8 KiB per wave
  static constexpr int kKm = kFrag + kWaves * kStage;
  static constexpr int kAdd = kKm + D * 4;
  static constexpr int kLpt = kAdd + D * 4;
  static constexpr int kTotal = kLpt + (kLptMax + 1) * 4;
};

// NORM: rowscale = 1 / (x_t . km + eps).  TOKENS (implies the job's q in xden): the token
// view of backward pass A: g = x_t M (x = dO, M = S^T), P = q~_t . g, z = q_t . km + eps,
// dz = -P / z^2, out = dq_t = g / z + dz km (without the denominator: out = g), and the
// per-row scalars 1/z_t, dz_t go to tokscal.  DEN (decoupled): the denominator rows are not
// the multiplied rows; they are read straight from global memory (NORM: z; TOKENS: z from q,
// P from q~ = q_rope, and the two gradients go to out = dq~ and out2 = dq).
template <bool NORM, bool TOKENS, bool PAD, bool DEN>
__global__ __launch_bounds__(kThreads) void rows32_kernel(Prob p, Rows32Job job0, Rows32Job job1,
                                                          int wgs_per_job, int chunk, int nchunks) {
  using LY = Rows32Layout;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const bool second = (int)blockIdx.x >= wgs_per_job;
  const Rows32Job& job = second ? job1 : job0;
  const int wg = second ? blockIdx.x - wgs_per_job : blockIdx.x;
  const int wg_nh = wg / nchunks, c = wg - wg_nh * nchunks;
  const int h = wg_nh % p.H;
  const int n = lpt_sequence(p, wg_nh / p.H, reinterpret_cast<int*>(smem + LY::kLpt));
  const int nh = n * p.H + h;
  int64_t bos, row0, rstride;
  int len;
  seq_range(p, n, bos, len);
  const int t_begin = c * chunk;
  if (t_begin >= len) return;
  const int t_end = min(len, t_begin + chunk);
  row_base(p, n, h, bos, row0, rstride);

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int ntok = lane & 31, kb = lane >> 5;
  const int dr = PAD ? job.dr : D, dc = PAD ? job.dc : D;
  float* frag = reinterpret_cast<float*>(smem);
  unsigned char* stage = smem + LY::kFrag + wave * LY::kStage;
  float* kmv = reinterpret_cast<float*>(smem + LY::kKm);
  float* addv = reinterpret_cast<float*>(smem + LY::kAdd);

  // x tile: 32 rows of 256 bytes = 512 chunks, 8 per lane, flat and coalesced
  auto load_tile = [&](f32x4(&dst)[8], const float* src, int tok0) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int q = lane + 64 * i, row = q >> 4, ch = q & 15;
      const int tok = tok0 + row;
      dst[i] = (tok < t_end && (!PAD || ch * 4 < dr))
                   ? stream_load<(FBLA_NT32 & 2) != 0, f32x4>(src + (row0 + (int64_t)tok * rstride) * dr + ch * 4)
                   : f32x4{0.f, 0.f, 0.f, 0.f};
    }
  };
  int t0 = t_begin + 32 * wave;
  f32x4 xr[8];
  if (t0 < t_end) load_tile(xr, job.x, t0);

  build_operand32(frag, job.mat + (int64_t)nh * dr * dc, job.ld_r, job.ld_c, 1.f, dr, dc);
  const int dkm = NORM ? dr : dc;  // length of km: the contracted side (output) or q's (token view)
  if (tid < D) {  // (both loads before either is used)
    const bool has_km = (NORM || TOKENS) && job.km && tid < dkm, has_add = job.addvec && tid < dc;
    const float kmx = has_km ? job.km[(int64_t)nh * dkm + tid] : 0.f;
    const float addx = has_add ? job.addvec[(int64_t)nh * dc + tid] * job.add_scale : 0.f;
    kmv[tid] = kmx;
    addv[tid] = addx;
  }
  __syncthreads();
  const bool with_den = (NORM || TOKENS) && job.km != nullptr;

  while (t0 < t_end) {
    wave_sync();  // the previous tile's staged output has been read out
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int q = lane + 64 * i;
      *reinterpret_cast<f32x4*>(stage + swz<256>(q >> 4, q & 15)) = xr[i];
    }
    const int tn = t0 + 32 * kWaves;
    if (tn < t_end) load_tile(xr, job.x, tn);
    wave_sync();

    f32x16 acc[2];
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[b][r] = 0.f;
    float z = 0.f;
#pragma unroll
    for (int sg = 0; sg < 8; ++sg) {
      // k-steps 4sg .. 4sg+3: x features 8sg + 2kb + {0,1} and 8sg + 4 + 2kb + {0,1}
      const f32x2 x01 = *reinterpret_cast<const f32x2*>(stage + swz<256>(ntok, 2 * sg) + 8 * kb);
      const f32x2 x23 = *reinterpret_cast<const f32x2*>(stage + swz<256>(ntok, 2 * sg + 1) + 8 * kb);
      const float xv[4] = {x01[0], x01[1], x23[0], x23[1]};
#pragma unroll
      for (int b = 0; b < 2; ++b) {
        const f32x4 a4 = *reinterpret_cast<const f32x4*>(frag + ((b * 8 + sg) * 64 + lane) * 4);
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[b] = mma(a4[e], xv[e], acc[b]);
      }
      if constexpr (NORM && !DEN) {
        const f32x2 k01 = *reinterpret_cast<const f32x2*>(kmv + 8 * sg + 2 * kb);
        const f32x2 k23 = *reinterpret_cast<const f32x2*>(kmv + 8 * sg + 4 + 2 * kb);
        z = fmaf(x01[0], k01[0], z);
        z = fmaf(x01[1], k01[1], z);
        z = fmaf(x23[0], k23[0], z);
        z = fmaf(x23[1], k23[1], z);
      }
    }
    // this lane: token ntok, output features 32*kb + 16*b + r
    float rs = 1.f, dz = 0.f;
    if constexpr (NORM) {
      if constexpr (DEN) {  // this lane's half of the plain row: one 128-byte line
        const int tok = min(t0 + ntok, t_end - 1);
        const float* drow = job.xden + (row0 + (int64_t)tok * rstride) * dr + 32 * kb;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          if (PAD && 32 * kb + 4 * i >= dr) continue;
          const f32x4 dv4 = *reinterpret_cast<const f32x4*>(drow + 4 * i);
          const f32x4 kv = *reinterpret_cast<const f32x4*>(kmv + 32 * kb + 4 * i);
#pragma unroll
          for (int j = 0; j < 4; ++j) z = fmaf(dv4[j], kv[j], z);
        }
      }
      z += __shfl_xor(z, 32);
      rs = 1.f / (z + p.eps);
    }
    if constexpr (TOKENS) {
      if (with_den) {
        // q row half of this lane straight from global memory (a full 128-byte line per lane)
        const int tok = min(t0 + ntok, t_end - 1);
        const int64_t roff = (row0 + (int64_t)tok * rstride) * dc + 32 * kb;
        const float* qrow = job.xden + roff;   // plain q: the denominator
        const float* nrow = job.xnum + roff;   // q~: the numerator
        float P = 0.f, zz = 0.f;
#pragma unroll
        for (int b = 0; b < 2; ++b)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            f32x4 qv = f32x4{0.f, 0.f, 0.f, 0.f}, nv = f32x4{0.f, 0.f, 0.f, 0.f};
            if (!PAD || 32 * kb + 16 * b + 4 * i < dc) {
              qv = *reinterpret_cast<const f32x4*>(qrow + 16 * b + 4 * i);
              nv = qv;
              if constexpr (DEN) nv = *reinterpret_cast<const f32x4*>(nrow + 16 * b + 4 * i);
            }
            const f32x4 kv = *reinterpret_cast<const f32x4*>(kmv + 32 * kb + 16 * b + 4 * i);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              P = fmaf(nv[j], acc[b][4 * i + j], P);
              zz = fmaf(qv[j], kv[j], zz);
            }
          }
        P += __shfl_xor(P, 32);
        zz += __shfl_xor(zz, 32);
        rs = 1.f / (zz + p.eps);
        dz = -P * rs * rs;
        if (kb == 0 && t0 + ntok < t_end) {
          const int64_t row = row0 + (int64_t)(t0 + ntok) * rstride;
          job.tokscal[row] = rs;
          job.tokscal[job.total_rows + row] = dz;
        }
      }
    }
    wave_sync();  // all lanes have read their x values; the staging tile is reused for out
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int c0 = 32 * kb + 16 * b + 4 * i;
        f32x4 w;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          float o = fmaf(acc[b][4 * i + j], rs, addv[c0 + j]);
          if constexpr (TOKENS && !DEN) o = fmaf(dz, kmv[c0 + j], o);
          w[j] = o;
        }
        *reinterpret_cast<f32x4*>(stage + swz<256>(ntok, c0 >> 2)) = w;
      }
    wave_sync();
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int q = lane + 64 * i, row = q >> 4, ch = q & 15;
      const int tok = t0 + row;
      if (tok < t_end && (!PAD || ch * 4 < dc))
        stream_store<(FBLA_NT32 & 4) != 0>(job.out + (row0 + (int64_t)tok * rstride) * dc + ch * 4,
                                           *reinterpret_cast<const f32x4*>(stage + swz<256>(row, ch)));
    }
    if constexpr (TOKENS && DEN) {  // the second gradient, dq = dz km, through the same tile
      wave_sync();
#pragma unroll
      for (int b = 0; b < 2; ++b)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int c0 = 32 * kb + 16 * b + 4 * i;
          *reinterpret_cast<f32x4*>(stage + swz<256>(ntok, c0 >> 2)) =
              f32x4{dz * kmv[c0], dz * kmv[c0 + 1], dz * kmv[c0 + 2], dz * kmv[c0 + 3]};
        }
      wave_sync();
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int q = lane + 64 * i, row = q >> 4, ch = q & 15;
        const int tok = t0 + row;
        if (tok < t_end && (!PAD || ch * 4 < dc))
          stream_store<(FBLA_NT32 & 4) != 0>(job.out2 + (row0 + (int64_t)tok * rstride) * dc + ch * 4,
                                             *reinterpret_cast<const f32x4*>(stage + swz<256>(row, ch)));
      }
    }
    t0 = tn;
  }
}

// ===========================================================================
// host side
// ===========================================================================
bool supported(const Prob& p) {
  if (wide(p)) return wide_supported(p);
  return p.DK >= 4 && p.DV >= 4 && p.DK <= D && p.DV <= D && p.DK % 4 == 0 && p.DV % 4 == 0;
}
static bool padded(const Prob& p) { return p.DK != D || p.DV != D; }

void state(const Prob& p, const float* kn, const float* v, const float* kd, float* partial,
           const float* tokscal, int64_t total_rows, int chunk, int nchunks, hipStream_t st, float* fin_mat,
           float* fin_vec) {
  if (wide(p)) return wide_state(p, kn, v, partial, tokscal, total_rows, chunk, nchunks, st, fin_mat, fin_vec);
  const dim3 grid((unsigned)((int64_t)p.N * p.H * nchunks)), block(kThreads);
  auto go = [&](auto kernel) {
    kernel<<<grid, block, 0, st>>>(p, kn, v, kd, partial, tokscal, tokscal ? total_rows : 0, fin_mat, fin_vec, chunk, nchunks);
  };
  // kd != kn: the decoupled operator (vector part from the plain rows)
  const int variant = (kd != kn ? 4 : 0) + (tokscal ? 2 : 0) + (padded(p) ? 1 : 0);
  switch (variant) {
    case 0: go(state32_kernel<false, false, false>); break;
    case 1: go(state32_kernel<false, false, true>); break;
    case 2: go(state32_kernel<false, true, false>); break;
    case 3: go(state32_kernel<false, true, true>); break;
    case 4: go(state32_kernel<true, false, false>); break;
    case 5: go(state32_kernel<true, false, true>); break;
    case 6: go(state32_kernel<true, true, false>); break;
    default: go(state32_kernel<true, true, true>); break;
  }
}

template <bool NORM, bool TOKENS, bool PAD, bool DEN>
static int launch_rows_k(const Prob& p, const Rows32Job& j0, const Rows32Job* j1, hipStream_t st) {
  auto kernel = rows32_kernel<NORM, TOKENS, PAD, DEN>;
  static thread_local bool configured = false;
  if (!configured) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, Rows32Layout::kTotal);
    if (e != hipSuccess) {
      set_error("cannot reserve %d bytes of LDS: %s", Rows32Layout::kTotal, hipGetErrorString(e));
      return kErrLaunch;
    }
    configured = true;
  }
  const int chunk = mfma::rows_chunk(p, D, D);
  const int nchunks = (int)cdiv64(p.L, chunk);
  const int wgs = (int)((int64_t)p.N * p.H * nchunks);
  const dim3 grid((unsigned)(j1 ? 2 * wgs : wgs)), block(kThreads);
  kernel<<<grid, block, Rows32Layout::kTotal, st>>>(p, j0, j1 ? *j1 : j0, wgs, chunk, nchunks);
  return kOk;
}

template <bool NORM, bool TOKENS, bool DEN = false>
static int launch_rows(const Prob& p, const Rows32Job& j0, const Rows32Job* j1, hipStream_t st) {
  if (padded(p)) return launch_rows_k<NORM, TOKENS, true, DEN>(p, j0, j1, st);
  return launch_rows_k<NORM, TOKENS, false, DEN>(p, j0, j1, st);
}

static Rows32Job convert(const mfma::RowsJob& j, int dr, int dc) {
  Rows32Job r;
  r.x = (const float*)j.x;
  r.xnum = nullptr;
  r.out2 = nullptr;
  r.xden = (const float*)j.xden;
  r.mat = j.mat;
  r.ld_r = j.ld_r;
  r.ld_c = j.ld_c;
  r.km = j.km;
  r.addvec = j.addvec;
  r.add_scale = j.add_scale;
  r.out = (float*)j.out;
  r.tokscal = nullptr;
  r.total_rows = 0;
  r.dr = dr;
  r.dc = dc;
  return r;
}

// dr, dc: the contracted and the output head dim of the job (of both jobs when there are two)
int rows(const Prob& p, const mfma::RowsJob& job, const mfma::RowsJob* job2, int dr, int dc, hipStream_t st) {
  if (wide(p)) return wide_rows(p, job, job2, dr, dc, st);
  const Rows32Job a = convert(job, dr, dc);
  if (job.xden && job.xden != job.x) return launch_rows<true, false, true>(p, a, nullptr, st);
  if (job.xden) return launch_rows<true, false>(p, a, nullptr, st);
  if (job2) {
    const Rows32Job b = convert(*job2, dr, dc);
    return launch_rows<false, false>(p, a, &b, st);
  }
  return launch_rows<false, false>(p, a, nullptr, st);
}

// qn / dqn: the rows of the numerator and their gradient (q_rope, dq_rope when decoupled, then
// qd = q and dqd = dq; otherwise qn == qd and dqd is not used)
int bwd_tokens(const Prob& p, const float* qn, const float* qd, const float* dout, const float* S,
               const float* km, float* dqn, float* dqd, float* tokscal, int64_t total_rows, hipStream_t st) {
  if (wide(p)) return wide_bwd_tokens(p, qn, dout, S, km, dqn, tokscal, total_rows, st);
  Rows32Job j;
  j.x = dout;
  j.xnum = qn;
  j.out2 = dqd;
  j.xden = qd;
  j.mat = S;  // M(r = dv, c = dk) = S[c][r]
  j.ld_r = 1;
  j.ld_c = p.DV;
  j.dr = p.DV;
  j.dc = p.DK;
  j.km = (p.flags & kNormalize) ? km : nullptr;
  j.addvec = nullptr;
  j.add_scale = 1.f;
  j.out = dqn;
  j.tokscal = tokscal;
  j.total_rows = total_rows;
  if (p.flags & kDecoupled) return launch_rows<false, true, true>(p, j, nullptr, st);
  return launch_rows<false, true>(p, j, nullptr, st);
}

}  // namespace mfma32
}  // namespace fbla
