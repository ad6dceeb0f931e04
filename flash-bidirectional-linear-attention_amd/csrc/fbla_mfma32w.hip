// MFMA kernels for fp32 inputs whose larger head dim is above 64: heads tiled 128 x 128 (head dims
// that are multiples of 4 up to 128, zero padding for the rest of the tile; true row lengths in
// memory).  The plain operator, with or without the denominator, dense and packed; the decoupled
// operator with such heads stays on the shape-generic kernels.  v_mfma_f32_32x32x2_f32, fp32
// throughout: one instruction covers two values of the contraction index and takes 64 cycles, and a
// token of a 128 x 128 head needs 8192 of them per compute unit and kernel against 1 KiB of rows, so
// these kernels are bound by the matrix unit at about 60 % of the HBM rate.
//
//  state32w_kernel   S_part = K^T V and sum_t k_t over a token chunk.  A workgroup of four waves
//                    shares the tokens; wave w owns the 64 x 64 block (w / 2, w % 2) of the state, so
//                    no wave's sum is added to another's.  A lane owns one feature of a token row
//                    (row loads are 128 contiguous bytes per half-wave, no transposition).  SCALED:
//                    the feature view of the backward (v = dO scaled by 1/z_t per row, vector part
//                    sum_t dz_t q_t).
//  rows32w_kernel    out_t = (x_t M) * rowscale_t + addvec, 128 x 128 M: the four waves share steps
//                    of 32 tokens staged in LDS; wave w keeps the fragments of output block w (32 of
//                    the 128 output columns: 64 registers) and multiplies every row of the step by
//                    them.  TOKENS: the token view of backward pass A (x = dO, M = S^T; then q.g, z,
//                    dz, dq and the per-row scalars; the four waves' parts of q.g and q.km meet in LDS).
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

typedef float f32x4 __attribute__((ext_vector_type(4)));

namespace {

constexpr int kThreads = 256;
constexpr int W = 128;  // tiled head dim

__device__ __forceinline__ f32x16 mma(float a, float b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
}

// ===========================================================================
// state kernel
// ===========================================================================
// Lane l = (f = l%32, kb = l/32); wave w = block (bk, bv).  A 16-token tile is eight k-steps; in
// k-step s the lane holds feature 64 bk + 32 a + f of the key row and 64 bv + 32 b + f of the value
// row of token 2s + kb (a, b = 0, 1).  All four waves walk the same tiles; two or three register
// buffers rotate.
template <bool SCALED, bool PAD>
__global__ __launch_bounds__(kThreads, 2) void state32w_kernel(
    Prob p, const float* __restrict__ kn, const float* __restrict__ v, float* __restrict__ partial,
    const float* __restrict__ tokscal, int64_t total_rows, float* fin_mat, float* fin_vec, int chunk,
    int nchunks) {
  __shared__ int lpt_lens[kLptMax + 1];
  const int dk = PAD ? p.DK : W, dv = PAD ? p.DV : W;  // row lengths in memory
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

  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int bk = wave >> 1, bv = wave & 1;
  if (PAD && (64 * bk >= dk || 64 * bv >= dv)) return;  // this wave's block lies in the padding
  const int f = lane & 31, kb = lane >> 5;
  // this lane's two key and two value features; one past the head dim is read from column 0 and
  // replaced by zero
  bool kok[2], vok[2];
  int kcol[2], vcol[2];
#pragma unroll
  for (int a = 0; a < 2; ++a) {
    kok[a] = !PAD || 64 * bk + 32 * a + f < dk;
    vok[a] = !PAD || 64 * bv + 32 * a + f < dv;
    kcol[a] = kok[a] ? 64 * bk + 32 * a + f : 0;
    vcol[a] = vok[a] ? 64 * bv + 32 * a + f : 0;
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
    float rz[SCALED ? 8 : 1], dz[SCALED ? 8 : 1];
  };
  const uint32_t kstep = (uint32_t)(rstride * dk), vstep = (uint32_t)(rstride * dv);
  // A tile that would cross the end of the chunk is moved back so that it ends there; the rows it
  // shares with the previous tile are zeroed before use.
  auto fetch = [&](Buf& b, int tok) {
    const int tb = min(tok, t_end - 16);
    const int64_t row = row0 + (int64_t)tb * rstride;
    const float* kp = kn + row * dk;
    const float* vp = v + row * dv;
#pragma unroll
    for (int s = 0; s < 8; ++s) {
      const size_t kro = (size_t)(2 * s + kb) * kstep, vro = (size_t)(2 * s + kb) * vstep;
#pragma unroll
      for (int a = 0; a < 2; ++a) {
        const float kx = stream_load<true, float>(kp + kro + kcol[a]);
        const float vx = stream_load<true, float>(vp + vro + vcol[a]);
        b.k[s][a] = kok[a] ? kx : 0.f;
        b.v[s][a] = vok[a] ? vx : 0.f;
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
      const int64_t r = row0 + (int64_t)min(t, t_end - 1) * rstride;
#pragma unroll
      for (int a = 0; a < 2; ++a) {
        const float kx = kn[r * dk + kcol[a]], vx = v[r * dv + vcol[a]];
        b.k[s][a] = ok && kok[a] ? kx : 0.f;
        b.v[s][a] = ok && vok[a] ? vx : 0.f;
      }
      if constexpr (SCALED) {
        const float rzx = tokscal[r], dzx = tokscal[total_rows + r];
        b.rz[s] = ok ? rzx : 0.f;
        b.dz[s] = ok ? dzx : 0.f;
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
        for (int a = 0; a < 2; ++a) b.k[s][a] = keep ? b.k[s][a] : 0.f;
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
        if constexpr (SCALED) ks[a] = fmaf(b.dz[s], b.k[s][a], ks[a]);
        else ks[a] += b.k[s][a];
      }
    }
  };
  int t0 = t_begin;
  if (t_end - t_begin < 16) {
    Buf b0;
    fetch_checked(b0, t0);
    compute(b0, t0, true);
  } else if constexpr (SCALED) {  // (the per-row scalars leave registers for two buffers)
    Buf b0, b1;
    fetch(b0, t0);
    while (true) {
      fetch(b1, t0 + 16);
      compute(b0, t0, false);
      t0 += 16;
      if (t0 >= t_end) break;
      fetch(b0, t0 + 16);
      compute(b1, t0, false);
      t0 += 16;
      if (t0 >= t_end) break;
    }
  } else {
    // three register buffers in rotation: the rows of two tiles are in flight while one is multiplied
    // (one tile is 2048 matrix cycles, less than a load takes under load)
    Buf b0, b1, b2;
    fetch(b0, t0);
    fetch(b1, t0 + 16);
    while (true) {
      fetch(b2, t0 + 32);
      compute(b0, t0, false);
      t0 += 16;
      if (t0 >= t_end) break;
      fetch(b0, t0 + 32);
      compute(b1, t0, false);
      t0 += 16;
      if (t0 >= t_end) break;
      fetch(b1, t0 + 32);
      compute(b2, t0, false);
      t0 += 16;
      if (t0 >= t_end) break;
    }
  }

  float* mat = fin_mat ? fin_mat + (int64_t)nh * dk * dv
                       : partial + ((int64_t)nh * nchunks + c) * (dk * dv + dk);
  float* vec = fin_mat ? (fin_vec ? fin_vec + (int64_t)nh * dk : nullptr) : mat + dk * dv;
  const float mscale = fin_mat ? seq_scale(p, len) : 1.f;
  const float vscale = fin_mat ? 1.0f / (float)len : 1.f;
  // the two waves of a key half hold the same vector part: the first one stores it
  reduce_store_block<1, false>(acc, ks, nullptr, mat + (64 * bk) * dv + 64 * bv, dv,
                               (vec && bv == 0) ? vec + 64 * bk : nullptr, mscale, vscale, 0, lane,
                               dk - 64 * bk, dv - 64 * bv);
}

// ===========================================================================
// rows kernel
// ===========================================================================
// C[m][n = token] = sum_k A[m][k] B[k][n], A = this wave's 32 columns of the operand M (registers),
// B = x (LDS).  The contraction index of k-step s = 4i + e and half-wave kb is feature
// r = 8i + 4kb + e: a lane's B values of four k-steps are one 16-byte read of the staged row.  Row
// m = 8g + 4kb' + j of the wave's block is output feature 32w + 16kb' + 4g + j: after the MFMAs a
// lane (token, kb') owns 16 consecutive output features.
struct RowsWJob {
  const float* x;       // [rows, dr] B operand
  const float* xnum;    // TOKENS: the rows q of the numerator and of the denominator
  const float* mat;     // operand M, element (r, c) at mat[nh*dr*dc + r*ld_r + c*ld_c]
  int ld_r, ld_c;
  const float* km;      // [NH, dr] (NORM) or [NH, dc] (TOKENS) mean key, or null
  const float* addvec;  // [NH, dc] added (times add_scale) to every output row, or null
  float add_scale;
  float* out;           // [rows, dc]
  float* tokscal;       // TOKENS: [2][total rows]: 1/z_t, dz_t
  int64_t total_rows;
  int dr, dc;           // row lengths of x and out in memory (<= 128, multiples of 4)
};

struct RowsWLayout {
  static constexpr int kTile = 32 * W * 4;      // one step: 32 rows of 512 bytes
  static constexpr int kX = 0;                  // x tiles [2]; the operand is staged here first
  static constexpr int kOut = 2 * kTile;        // output staging
  static constexpr int kKm = kOut + kTile;
  static constexpr int kAdd = kKm + W * 4;
  static constexpr int kPz = kAdd + W * 4;      // [wave][32 tokens] (q.g, q.km)
  static constexpr int kLpt = kPz + 4 * 32 * 8;
  static constexpr int kTotal = kLpt + (kLptMax + 1) * 4;
  static_assert(3 * kTotal <= 160 * 1024, "three workgroups per CU");
};

// 16-byte chunk `ch` (0..31) of row `row` of a tile with 512-byte rows
__device__ __forceinline__ int swz512(int row, int ch) { return row * 512 + ((ch ^ (row & 31)) << 4); }

template <bool NORM, bool TOKENS, bool PAD>
__global__ __launch_bounds__(kThreads, 2) void rows32w_kernel(Prob p, RowsWJob job0, RowsWJob job1,
                                                              int wgs_per_job, int chunk, int nchunks) {
  using LY = RowsWLayout;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const bool second = (int)blockIdx.x >= wgs_per_job;
  const RowsWJob& job = second ? job1 : job0;
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
  const int dr = PAD ? job.dr : W, dc = PAD ? job.dc : W;
  unsigned char* xt = smem + LY::kX;
  unsigned char* ot = smem + LY::kOut;
  float* kmv = reinterpret_cast<float*>(smem + LY::kKm);
  float* addv = reinterpret_cast<float*>(smem + LY::kAdd);
  float* pz = reinterpret_cast<float*>(smem + LY::kPz);

  // a step's 32 rows of 512 bytes = 1024 chunks, 4 per thread, flat and coalesced
  auto load_step = [&](f32x4(&dst)[4], const float* src, int tok0) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int q = tid + kThreads * i, row = q >> 5, ch = q & 31;
      const int tok = tok0 + row;
      dst[i] = (tok < t_end && (!PAD || ch * 4 < dr))
                   ? stream_load<true, f32x4>(src + (row0 + (int64_t)tok * rstride) * dr + ch * 4)
                   : f32x4{0.f, 0.f, 0.f, 0.f};
    }
  };
  f32x4 xr[4];
  load_step(xr, job.x, t_begin);

  // ---- the operand: two passes of two 32-column blocks through the tile area; wave w keeps block w
  f32x4 areg[16];
  {
    const float* mat = job.mat + (int64_t)nh * dr * dc;
    const bool c_fast = job.ld_c == 1;  // walk the matrix along its contiguous direction
    float* frag = reinterpret_cast<float*>(xt);
#pragma unroll 1
    for (int pass = 0; pass < 2; ++pass) {
      constexpr int kPer = W * 64 / kThreads;  // 32 elements per thread and pass
      float val[kPer];
#pragma unroll
      for (int i = 0; i < kPer; ++i) {
        const int e = tid + i * kThreads;
        const int r = c_fast ? e >> 6 : e & 127, cc = 64 * pass + (c_fast ? e & 63 : e >> 7);
        const bool in = r < dr && cc < dc;
        val[i] = mat[in ? (int64_t)r * job.ld_r + (int64_t)cc * job.ld_c : 0];
        val[i] = in ? val[i] : 0.f;
      }
      if (pass) __syncthreads();  // the first pass's fragments have been read
#pragma unroll
      for (int i = 0; i < kPer; ++i) {
        const int e = tid + i * kThreads;
        const int r = c_fast ? e >> 6 : e & 127, ccl = c_fast ? e & 63 : e >> 7;
        const int ii = r >> 3, kbr = (r >> 2) & 1, ee = r & 3;
        const int b = ccl >> 5, kbp = (ccl >> 4) & 1, g = (ccl >> 2) & 3, j = ccl & 3;
        const int m = 8 * g + 4 * kbp + j;
        frag[(((b * 16 + ii) * 64) + m + 32 * kbr) * 4 + ee] = val[i];
      }
      __syncthreads();
      if ((wave >> 1) == pass) {
#pragma unroll
        for (int i = 0; i < 16; ++i)
          areg[i] = *reinterpret_cast<const f32x4*>(frag + (((wave & 1) * 16 + i) * 64 + lane) * 4);
      }
    }
    // vectors: km along the contracted side (NORM: z = x . km) or the output side (TOKENS: z = q . km)
    const int dkm = NORM ? dr : dc;
    if (tid < W) {
      const bool has_km = (NORM || TOKENS) && job.km && tid < dkm, has_add = job.addvec && tid < dc;
      const float kmx = has_km ? job.km[(int64_t)nh * dkm + tid] : 0.f;
      const float addx = has_add ? job.addvec[(int64_t)nh * dc + tid] * job.add_scale : 0.f;
      kmv[tid] = kmx;
      addv[tid] = addx;
    }
    __syncthreads();  // the fragments have left the tile area
  }
  const bool with_den = (NORM || TOKENS) && job.km != nullptr;
  const int col0 = 32 * wave + 16 * kb;  // this lane's 16 output features

  int buf = 0;
  for (int t0 = t_begin; t0 < t_end; t0 += 32, buf ^= 1) {
    unsigned char* xb = xt + buf * LY::kTile;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int q = tid + kThreads * i;
      *reinterpret_cast<f32x4*>(xb + swz512(q >> 5, q & 31)) = xr[i];
    }
    load_step(xr, job.x, t0 + 32);
    // TOKENS: this lane's 16 features of its token's q row (64 contiguous bytes), requested early
    f32x4 qv[4];
    if constexpr (TOKENS) {
      const int tok = min(t0 + ntok, t_end - 1);
      const float* qrow = job.xnum + (row0 + (int64_t)tok * rstride) * dc + col0;
#pragma unroll
      for (int i = 0; i < 4; ++i)
        qv[i] = (!PAD || col0 + 4 * i < dc) ? *reinterpret_cast<const f32x4*>(qrow + 4 * i) : f32x4{0.f, 0.f, 0.f, 0.f};
    }
    __syncthreads();  // the step is staged (and the previous step's staged output has left)

    f32x16 acc;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0.f;
    float z = 0.f;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const f32x4 xv = *reinterpret_cast<const f32x4*>(xb + swz512(ntok, 2 * i + kb));
#pragma unroll
      for (int e = 0; e < 4; ++e) acc = mma(areg[i][e], xv[e], acc);
      if constexpr (NORM) {
        const f32x4 kv = *reinterpret_cast<const f32x4*>(kmv + 8 * i + 4 * kb);
#pragma unroll
        for (int e = 0; e < 4; ++e) z = fmaf(xv[e], kv[e], z);
      }
    }
    float rs = 1.f, dz = 0.f;
    if constexpr (NORM) {
      z += __shfl_xor(z, 32);
      rs = 1.f / (z + p.eps);
    }
    if constexpr (TOKENS) {
      if (with_den) {
        float P = 0.f, zz = 0.f;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const f32x4 kv = *reinterpret_cast<const f32x4*>(kmv + col0 + 4 * i);
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            P = fmaf(qv[i][j], acc[4 * i + j], P);
            zz = fmaf(qv[i][j], kv[j], zz);
          }
        }
        P += __shfl_xor(P, 32);
        zz += __shfl_xor(zz, 32);
        if (kb == 0) *reinterpret_cast<float2*>(&pz[2 * (wave * 32 + ntok)]) = float2{P, zz};
        __syncthreads();
        P = 0.f;
        zz = 0.f;
#pragma unroll
        for (int w = 0; w < 4; ++w) {  // the four parts in wave order: the same sum in every wave
          const float2 part = *reinterpret_cast<const float2*>(&pz[2 * (w * 32 + ntok)]);
          P += part.x;
          zz += part.y;
        }
        rs = 1.f / (zz + p.eps);
        dz = -P * rs * rs;
        if (wave == 0 && kb == 0 && t0 + ntok < t_end) {
          const int64_t row = row0 + (int64_t)(t0 + ntok) * rstride;
          job.tokscal[row] = rs;
          job.tokscal[job.total_rows + row] = dz;
        }
      }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f32x4 w;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        float o = fmaf(acc[4 * i + j], rs, addv[col0 + 4 * i + j]);
        if constexpr (TOKENS) o = fmaf(dz, kmv[col0 + 4 * i + j], o);
        w[j] = o;
      }
      *reinterpret_cast<f32x4*>(ot + swz512(ntok, (col0 >> 2) + i)) = w;
    }
    __syncthreads();  // whole output rows are staged (and every wave has read the x tile and pz)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int q = tid + kThreads * i, row = q >> 5, ch = q & 31;
      const int tok = t0 + row;
      if (tok < t_end && (!PAD || ch * 4 < dc))
        stream_store<true>(job.out + (row0 + (int64_t)tok * rstride) * dc + ch * 4,
                           *reinterpret_cast<const f32x4*>(ot + swz512(row, ch)));
    }
  }
}

bool wide_padded(const Prob& p) { return p.DK != W || p.DV != W; }

// Tokens per workgroup of the row kernel: two rounds of the workgroups that fit the 256 compute
// units (two per unit), at least 128 tokens, whole steps.
int wide_rows_chunk(const Prob& p) {
  const int64_t nh = (int64_t)p.N * p.H;
  int64_t nchunks = (256 * 2 * 2) / (nh > 0 ? nh : 1);
  if (nchunks < 1) nchunks = 1;
  int64_t chunk = cdiv64(p.L, nchunks);
  if (chunk < 128) chunk = 128;
  return (int)(cdiv64(chunk, 32) * 32);
}

template <bool NORM, bool TOKENS, bool PAD>
int launch_rows_w(const Prob& p, const RowsWJob& j0, const RowsWJob* j1, hipStream_t st) {
  auto kernel = rows32w_kernel<NORM, TOKENS, PAD>;
  static thread_local bool configured = false;
  if (!configured) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, RowsWLayout::kTotal);
    if (e != hipSuccess) {
      set_error("cannot reserve %d bytes of LDS: %s", RowsWLayout::kTotal, hipGetErrorString(e));
      return kErrLaunch;
    }
    configured = true;
  }
  const int chunk = wide_rows_chunk(p);
  const int nchunks = (int)cdiv64(p.L, chunk);
  const int wgs = (int)((int64_t)p.N * p.H * nchunks);
  const dim3 grid((unsigned)(j1 ? 2 * wgs : wgs)), block(kThreads);
  kernel<<<grid, block, RowsWLayout::kTotal, st>>>(p, j0, j1 ? *j1 : j0, wgs, chunk, nchunks);
  return kOk;
}

template <bool NORM, bool TOKENS>
int launch_rows_wp(const Prob& p, const RowsWJob& j0, const RowsWJob* j1, hipStream_t st) {
  if (wide_padded(p)) return launch_rows_w<NORM, TOKENS, true>(p, j0, j1, st);
  return launch_rows_w<NORM, TOKENS, false>(p, j0, j1, st);
}

RowsWJob convert_w(const mfma::RowsJob& j, int dr, int dc) {
  RowsWJob r;
  r.x = (const float*)j.x;
  r.xnum = nullptr;
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

}  // namespace

// heads with a side above 64: the plain operator only
bool wide(const Prob& p) { return p.DK > 64 || p.DV > 64; }
bool wide_supported(const Prob& p) {
  return !(p.flags & kDecoupled) && p.DK >= 4 && p.DV >= 4 && p.DK <= W && p.DV <= W && p.DK % 4 == 0 &&
         p.DV % 4 == 0 && !(p.cu && p.H > 65536);
}

void wide_state(const Prob& p, const float* kn, const float* v, float* partial, const float* tokscal,
                int64_t total_rows, int chunk, int nchunks, hipStream_t st, float* fin_mat, float* fin_vec) {
  const dim3 grid((unsigned)((int64_t)p.N * p.H * nchunks)), block(kThreads);
  auto go = [&](auto kernel) {
    kernel<<<grid, block, 0, st>>>(p, kn, v, partial, tokscal, tokscal ? total_rows : 0, fin_mat, fin_vec, chunk,
                                   nchunks);
  };
  switch ((tokscal ? 2 : 0) + (wide_padded(p) ? 1 : 0)) {
    case 0: go(state32w_kernel<false, false>); break;
    case 1: go(state32w_kernel<false, true>); break;
    case 2: go(state32w_kernel<true, false>); break;
    default: go(state32w_kernel<true, true>); break;
  }
}

// dr, dc: the contracted and the output head dim of the job (of both jobs when there are two)
int wide_rows(const Prob& p, const mfma::RowsJob& job, const mfma::RowsJob* job2, int dr, int dc, hipStream_t st) {
  const RowsWJob a = convert_w(job, dr, dc);
  if (job.xden) return launch_rows_wp<true, false>(p, a, nullptr, st);
  if (job2) {
    const RowsWJob b = convert_w(*job2, dr, dc);
    return launch_rows_wp<false, false>(p, a, &b, st);
  }
  return launch_rows_wp<false, false>(p, a, nullptr, st);
}

int wide_bwd_tokens(const Prob& p, const float* q, const float* dout, const float* S, const float* km, float* dq,
                    float* tokscal, int64_t total_rows, hipStream_t st) {
  RowsWJob j;
  j.x = dout;
  j.xnum = q;
  j.mat = S;  // M(r = dv, c = dk) = S[c][r]
  j.ld_r = 1;
  j.ld_c = p.DV;
  j.dr = p.DV;
  j.dc = p.DK;
  j.km = (p.flags & kNormalize) ? km : nullptr;
  j.addvec = nullptr;
  j.add_scale = 1.f;
  j.out = dq;
  j.tokscal = tokscal;
  j.total_rows = total_rows;
  return launch_rows_wp<false, true>(p, j, nullptr, st);
}

}  // namespace mfma32
}  // namespace fbla
