// Shape-generic kernels: any DK, DV in [1,128], fp16 / bf16 / fp32 inputs, dense
// [B,H,L,D] or packed [T,H,D] layout.  They stage token tiles through LDS as
// fp32 and use plain FMA arithmetic; the MFMA kernels in fbla_mfma.hip take over
// for the 16-bit head dims they cover.  All cross-workgroup reductions are
// two-stage and fixed-order (no atomics), so results are run-to-run identical.
//
// Replaces the Triton kernels of flash_bla/ops/linear_attn/fused.py:26-347,
// decoupled.py:27-408, varlen.py:30-332 and simple_la/fused.py:26-426.
#include <algorithm>

#include "fbla_kernels.h"

namespace fbla {
namespace generic {

constexpr int kThreads = 256;
constexpr int kTile = 32;   // tokens per LDS stage
constexpr int kLd = 129;    // LDS row pitch in floats (128 + 1: conflict-free column walks)

// ---------------------------------------------------------------------------
// helpers
// ---------------------------------------------------------------------------

// Copy rows [t0, t0+nvalid) x [0,D) of X into dst[kTile][kLd] as fp32, zero-filling
// the rest of the [kTile][Dpad] rectangle.
// BATCH: loads in flight per thread and tensor (16 = the whole tile at once).  Backward pass A,
// whose accumulators leave fewer registers, takes 8: with 16 it runs at half the occupancy and half
// the speed.
template <typename T, int BATCH = 16>
__device__ __forceinline__ void load_tile(float* dst, const T* __restrict__ X, int64_t row0,
                                          int64_t rstride, int D, int Dpad, int t0, int nvalid) {
  // A batch's elements are all requested before the first is stored (clamped addresses instead
  // of branches: a loop of guarded loads waits for every single one).  Dpad <= 128.
  constexpr int kPer = kTile * 128 / kThreads;
  static_assert(kPer % BATCH == 0, "whole batches");
  const int n = kTile * Dpad;
#pragma unroll
  for (int b0 = 0; b0 < kPer; b0 += BATCH) {
    if (b0 * kThreads >= n) break;  // uniform: narrower tiles need fewer batches
    float x[BATCH];
#pragma unroll
    for (int u = 0; u < BATCH; ++u) {
      const int i = threadIdx.x + (b0 + u) * kThreads, t = i / Dpad, d = i - t * Dpad;
      const bool in = i < n && t < nvalid && d < D;
      x[u] = to_f32(X[in ? (row0 + (int64_t)(t0 + t) * rstride) * D + d : 0]);
      x[u] = in ? x[u] : 0.f;
    }
#pragma unroll
    for (int u = 0; u < BATCH; ++u) {
      const int i = threadIdx.x + (b0 + u) * kThreads, t = i / Dpad, d = i - t * Dpad;
      if (i < n) dst[t * kLd + d] = x[u];
    }
  }
}

// acc[r][c] += sum_t Ls[t][ty+16r] * Rs[t][tx+16c]  (token-contracted outer products)
template <int M>
__device__ __forceinline__ void outer_accumulate(float (&acc)[M][M], const float* Ls,
                                                 const float* Rs, int tx, int ty) {
#pragma unroll 4
  for (int t = 0; t < kTile; ++t) {
    float a[M], b[M];
#pragma unroll
    for (int r = 0; r < M; ++r) a[r] = Ls[t * kLd + ty + 16 * r];
#pragma unroll
    for (int c = 0; c < M; ++c) b[c] = Rs[t * kLd + tx + 16 * c];
#pragma unroll
    for (int r = 0; r < M; ++r)
#pragma unroll
      for (int c = 0; c < M; ++c) acc[r][c] = fmaf(a[r], b[c], acc[r][c]);
  }
}

// acc[i][j] = sum_r Xs[tg+8i][r] * Mat[r][lane+32j]   (token rows times a small matrix)
template <int UNROLL = 4>
__device__ __forceinline__ void rows_times_matrix(float (&acc)[4][4], const float* Xs,
                                                  const float* __restrict__ Mat, int R, int C,
                                                  int tg, int lane) {
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;
  // (clamped column instead of a branch, UNROLL rows per trip: their loads of the matrix are in
  // flight together - guarded loads in a rolled loop wait for every single one)
#pragma unroll UNROLL
  for (int r = 0; r < R; ++r) {
    float m[4], x[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int c = lane + 32 * j;
      m[j] = Mat[(int64_t)r * C + (c < C ? c : 0)];
      m[j] = c < C ? m[j] : 0.f;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) x[i] = Xs[(tg + 8 * i) * kLd + r];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(x[i], m[j], acc[i][j]);
  }
}

template <int M>
__device__ __forceinline__ void write_partial(float* dst, const float (&acc)[M][M], int DK, int DV,
                                              int tx, int ty) {
#pragma unroll
  for (int r = 0; r < M; ++r)
#pragma unroll
    for (int c = 0; c < M; ++c) {
      int dk = ty + 16 * r, dv = tx + 16 * c;
      if (dk < DK && dv < DV) dst[dk * DV + dv] = acc[r][c];
    }
}

// ---------------------------------------------------------------------------
// forward, stage 1: per (sequence, head, token chunk) partial K~^T V and sum_t k_t
// ---------------------------------------------------------------------------
template <typename T, int M>
__global__ __launch_bounds__(kThreads) void state_partial_kernel(
    Prob p, const T* __restrict__ kn, const T* __restrict__ v, const T* __restrict__ kd,
    float* __restrict__ partial, int chunk, int nchunks) {
  __shared__ float Ls[kTile * kLd];
  __shared__ float Rs[kTile * kLd];
  __shared__ float Cs[kTile * kLd];
  const int nh = blockIdx.x / nchunks, c = blockIdx.x - nh * nchunks;
  const int n = nh / p.H, h = nh - n * p.H;
  int64_t bos, row0, rstride;
  int len;
  seq_range(p, n, bos, len);
  const int t_begin = c * chunk;
  if (t_begin >= len) return;
  const int t_end = min(len, t_begin + chunk);
  row_base(p, n, h, bos, row0, rstride);

  const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
  const int DK = p.DK, DV = p.DV, Dpad = 16 * M;
  const bool split = p.flags & kDecoupled;
  float acc[M][M];
#pragma unroll
  for (int r = 0; r < M; ++r)
#pragma unroll
    for (int cc = 0; cc < M; ++cc) acc[r][cc] = 0.f;
  float ksum = 0.f;

  for (int t0 = t_begin; t0 < t_end; t0 += kTile) {
    const int nvalid = min(kTile, t_end - t0);
    load_tile(Ls, kn, row0, rstride, DK, Dpad, t0, nvalid);
    load_tile(Rs, v, row0, rstride, DV, Dpad, t0, nvalid);
    if (split) load_tile(Cs, kd, row0, rstride, DK, Dpad, t0, nvalid);
    __syncthreads();
    outer_accumulate<M>(acc, Ls, Rs, tx, ty);
    if ((int)threadIdx.x < DK) {
      const float* src = split ? Cs : Ls;
      for (int t = 0; t < kTile; ++t) ksum += src[t * kLd + threadIdx.x];
    }
    __syncthreads();
  }
  float* dst = partial + (int64_t)blockIdx.x * (DK * DV + DK);
  write_partial<M>(dst, acc, DK, DV, tx, ty);
  if ((int)threadIdx.x < DK) dst[DK * DV + threadIdx.x] = ksum;
}

// ---------------------------------------------------------------------------
// stage 2 (forward and backward): fixed-order sum of the chunk partials.
//   mat[dk][dv] = scale_n * sum_c partial_c ;  mat_t = its transpose (optional)
//   vec[dk]     = (1/len) * sum_c partial_vec_c
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(kThreads) void state_reduce_kernel(
    Prob p, const float* __restrict__ partial, int chunk, int nchunks, float* __restrict__ mat,
    float* __restrict__ mat_t, float* __restrict__ vec, int blocks_per_head) {
  const int nh = blockIdx.x / blocks_per_head, blk = blockIdx.x - nh * blocks_per_head;
  const int n = nh / p.H;
  int64_t bos;
  int len;
  seq_range(p, n, bos, len);
  const int DK = p.DK, DV = p.DV, E = DK * DV, stride = E + DK;
  const int e = blk * kThreads + threadIdx.x;
  if (e >= stride) return;
  const int nvalid = len > 0 ? min(nchunks, (len + chunk - 1) / chunk) : 0;
  const float* src = partial + partial_slot(p, n, nh - n * p.H, 0, nchunks) * stride + e;
  const int64_t cstride = (int64_t)stride * partial_step(p);  // between consecutive chunks
  // fixed order: chunk 0, 1, 2, ... (four independent loads in flight at a time)
  float a = 0.f;
  int c = 0;
  for (; c + 4 <= nvalid; c += 4) {
    const float x0 = src[c * cstride], x1 = src[(c + 1) * cstride];
    const float x2 = src[(c + 2) * cstride], x3 = src[(c + 3) * cstride];
    a = (((a + x0) + x1) + x2) + x3;
  }
  for (; c < nvalid; ++c) a += src[c * cstride];
  if (e < E) {
    a *= seq_scale(p, len);
    mat[(int64_t)nh * E + e] = a;
    if (mat_t) {
      const int dk = e / DV, dv = e - dk * DV;
      mat_t[(int64_t)nh * E + dv * DK + dk] = a;
    }
  } else if (vec) {
    vec[(int64_t)nh * DK + (e - E)] = len > 0 ? a / (float)len : 0.f;
  }
}

__global__ __launch_bounds__(kThreads) void transpose_state_kernel(const float* __restrict__ mat,
                                                                   float* __restrict__ mat_t,
                                                                   int DK, int DV) {
  const int64_t base = (int64_t)blockIdx.x * DK * DV;
  for (int e = threadIdx.x; e < DK * DV; e += kThreads) {
    int dk = e / DV, dv = e - dk * DV;
    mat_t[base + dv * DK + dk] = mat[base + e];
  }
}

// ---------------------------------------------------------------------------
// forward, stage 3: o_t = (q~_t S) / (q_t . km + eps)
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(kThreads) void output_kernel(
    Prob p, const T* __restrict__ qn, const T* __restrict__ qd, const float* __restrict__ S,
    const float* __restrict__ km, T* __restrict__ o, int ntiles) {
  __shared__ float Xs[kTile * kLd];
  __shared__ float Ds[kTile * kLd];
  __shared__ float zs[kTile];
  const int nh = blockIdx.x / ntiles, tile = blockIdx.x - nh * ntiles;
  const int n = nh / p.H, h = nh - n * p.H;
  int64_t bos, row0, rstride;
  int len;
  seq_range(p, n, bos, len);
  const int t0 = tile * kTile;
  if (t0 >= len) return;
  const int nvalid = min(kTile, len - t0);
  row_base(p, n, h, bos, row0, rstride);
  const int DK = p.DK, DV = p.DV;
  const bool normalize = p.flags & kNormalize;
  const bool split = p.flags & kDecoupled;

  load_tile(Xs, qn, row0, rstride, DK, DK, t0, nvalid);
  if (split && normalize) load_tile(Ds, qd, row0, rstride, DK, DK, t0, nvalid);
  __syncthreads();
  if (threadIdx.x < kTile) {
    float z = 1.f;
    if (normalize) {
      const float* src = split ? Ds : Xs;
      const float* kmh = km + (int64_t)nh * DK;
      z = 0.f;
      for (int r = 0; r < DK; ++r) z = fmaf(src[threadIdx.x * kLd + r], kmh[r], z);
      z += p.eps;
    }
    zs[threadIdx.x] = z;
  }
  __syncthreads();
  const int tg = threadIdx.x >> 5, lane = threadIdx.x & 31;
  float acc[4][4];
  rows_times_matrix(acc, Xs, S + (int64_t)nh * DK * DV, DK, DV, tg, lane);
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int t = tg + 8 * i;
    if (t >= nvalid) continue;
    const float rz = 1.0f / zs[t];
    T* dst = o + (row0 + (int64_t)(t0 + t) * rstride) * DV;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int c = lane + 32 * j;
      if (c < DV) dst[c] = from_f32<T>(acc[i][j] * rz);
    }
  }
}

// ---------------------------------------------------------------------------
// backward, pass A: reads q~, q, dO (+S, S^T, km); writes dq~ (and dq when
// decoupled) and per-chunk partials of dS = sum_t (q~_t/z_t)^T dO_t and
// dkm = sum_t dz_t q_t, with dz_t = -(o_t.dO_t)/z_t and o_t recomputed from q~_t S.
// ---------------------------------------------------------------------------
template <typename T, int M>
__global__ __launch_bounds__(kThreads) void bwd_a_kernel(
    Prob p, const T* __restrict__ qn, const T* __restrict__ qd, const T* __restrict__ dout,
    const float* __restrict__ S, const float* __restrict__ St, const float* __restrict__ km,
    T* __restrict__ dqn, T* __restrict__ dqd, float* __restrict__ partial, int chunk,
    int nchunks) {
  __shared__ float Qn[kTile * kLd];
  __shared__ float Qd[kTile * kLd];
  __shared__ float Gs[kTile * kLd];
  __shared__ float zs[kTile];
  __shared__ float dzs[kTile];
  __shared__ float Ps[kTile];
  const int nh = blockIdx.x / nchunks, c = blockIdx.x - nh * nchunks;
  const int n = nh / p.H, h = nh - n * p.H;
  int64_t bos, row0, rstride;
  int len;
  seq_range(p, n, bos, len);
  const int t_begin = c * chunk;
  if (t_begin >= len) return;
  const int t_end = min(len, t_begin + chunk);
  row_base(p, n, h, bos, row0, rstride);

  const int DK = p.DK, DV = p.DV, Dpad = 16 * M;
  const bool normalize = p.flags & kNormalize;
  const bool split = p.flags & kDecoupled;
  const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
  const int tg = threadIdx.x >> 5, lane = threadIdx.x & 31;
  const float* Sh = S + (int64_t)nh * DK * DV;
  const float* Sth = St + (int64_t)nh * DK * DV;
  const float* kmh = km + (int64_t)nh * DK;

  float acc[M][M];
#pragma unroll
  for (int r = 0; r < M; ++r)
#pragma unroll
    for (int cc = 0; cc < M; ++cc) acc[r][cc] = 0.f;
  float dkm = 0.f;

  for (int t0 = t_begin; t0 < t_end; t0 += kTile) {
    const int nvalid = min(kTile, t_end - t0);
    load_tile<T, 8>(Qn, qn, row0, rstride, DK, Dpad, t0, nvalid);
    load_tile<T, 8>(Gs, dout, row0, rstride, DV, Dpad, t0, nvalid);
    if (split) load_tile<T, 8>(Qd, qd, row0, rstride, DK, Dpad, t0, nvalid);
    __syncthreads();
    const float* Qden = split ? Qd : Qn;
    float u[4][4];
    if (normalize) {
      if (threadIdx.x < kTile) {
        float z = 0.f;
        for (int r = 0; r < DK; ++r) z = fmaf(Qden[threadIdx.x * kLd + r], kmh[r], z);
        zs[threadIdx.x] = (int)threadIdx.x < nvalid ? z + p.eps : 1.0f;  // padding rows: dz = 0
      }
      // P_t = (q~_t S) . dO_t
      rows_times_matrix<2>(u, Qn, Sh, DK, DV, tg, lane);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int t = tg + 8 * i;
        float part = 0.f;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int cc = lane + 32 * j;
          if (cc < DV) part = fmaf(u[i][j], Gs[t * kLd + cc], part);
        }
#pragma unroll
        for (int off = 16; off > 0; off >>= 1) part += __shfl_xor(part, off, 32);
        if (lane == 0) Ps[t] = part;
      }
      __syncthreads();
      if (threadIdx.x < kTile) {
        const float z = zs[threadIdx.x];
        dzs[threadIdx.x] = -Ps[threadIdx.x] / (z * z);
      }
      __syncthreads();
    }
    // dq~_t = dO_t S^T / z_t (+ dz_t km when q~ == q)
    rows_times_matrix<2>(u, Gs, Sth, DV, DK, tg, lane);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int t = tg + 8 * i;
      if (t >= nvalid) continue;
      const float rz = normalize ? 1.0f / zs[t] : 1.0f;
      const float dz = normalize ? dzs[t] : 0.f;
      const int64_t roff = (row0 + (int64_t)(t0 + t) * rstride) * DK;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int cc = lane + 32 * j;
        if (cc >= DK) continue;
        float g = u[i][j] * rz;
        const float den = normalize ? dz * kmh[cc] : 0.f;
        if (split) {
          dqd[roff + cc] = from_f32<T>(den);
        } else {
          g += den;
        }
        dqn[roff + cc] = from_f32<T>(g);
      }
    }
    if (normalize) {
      if ((int)threadIdx.x < DK) {
        for (int t = 0; t < kTile; ++t) dkm = fmaf(dzs[t], Qden[t * kLd + threadIdx.x], dkm);
      }
      __syncthreads();
      for (int i = threadIdx.x; i < kTile * Dpad; i += kThreads) {
        int t = i / Dpad, d = i - t * Dpad;
        Qn[t * kLd + d] *= 1.0f / zs[t];
      }
      __syncthreads();
    }
    outer_accumulate<M>(acc, Qn, Gs, tx, ty);
    __syncthreads();
  }
  float* dst = partial + (int64_t)blockIdx.x * (DK * DV + DK);
  write_partial<M>(dst, acc, DK, DV, tx, ty);
  if ((int)threadIdx.x < DK) dst[DK * DV + threadIdx.x] = dkm;
}

// ---------------------------------------------------------------------------
// backward, pass B: dk~_t = v_t (s dS)^T (+ dkm/L when k~ == k), dv_t = k~_t (s dS),
// and dk_t = dkm/L for every row when decoupled.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(kThreads) void bwd_b_kernel(
    Prob p, const T* __restrict__ kn, const T* __restrict__ v, const float* __restrict__ dS,
    const float* __restrict__ dSt, const float* __restrict__ dkm, T* __restrict__ dkn,
    T* __restrict__ dkd, T* __restrict__ dv, int ntiles, float dkm_scale) {
  __shared__ float Ks[kTile * kLd];
  __shared__ float Vs[kTile * kLd];
  const int nh = blockIdx.x / ntiles, tile = blockIdx.x - nh * ntiles;
  const int n = nh / p.H, h = nh - n * p.H;
  int64_t bos, row0, rstride;
  int len;
  seq_range(p, n, bos, len);
  const int t0 = tile * kTile;
  if (t0 >= len) return;
  const int nvalid = min(kTile, len - t0);
  row_base(p, n, h, bos, row0, rstride);
  const int DK = p.DK, DV = p.DV;
  const bool normalize = p.flags & kNormalize;
  const bool split = p.flags & kDecoupled;
  const float* dSh = dS + (int64_t)nh * DK * DV;
  const float* dSth = dSt + (int64_t)nh * DK * DV;
  const float* dkmh = dkm + (int64_t)nh * DK;

  load_tile(Ks, kn, row0, rstride, DK, DK, t0, nvalid);
  load_tile(Vs, v, row0, rstride, DV, DV, t0, nvalid);
  __syncthreads();
  const int tg = threadIdx.x >> 5, lane = threadIdx.x & 31;
  float acc[4][4];
  rows_times_matrix(acc, Vs, dSth, DV, DK, tg, lane);
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int t = tg + 8 * i;
    if (t >= nvalid) continue;
    const int64_t roff = (row0 + (int64_t)(t0 + t) * rstride) * DK;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int cc = lane + 32 * j;
      if (cc >= DK) continue;
      float g = acc[i][j];
      const float den = normalize ? dkmh[cc] * dkm_scale : 0.f;
      if (split) {
        dkd[roff + cc] = from_f32<T>(den);
      } else {
        g += den;
      }
      dkn[roff + cc] = from_f32<T>(g);
    }
  }
  rows_times_matrix(acc, Ks, dSh, DK, DV, tg, lane);
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int t = tg + 8 * i;
    if (t >= nvalid) continue;
    const int64_t roff = (row0 + (int64_t)(t0 + t) * rstride) * DV;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int cc = lane + 32 * j;
      if (cc < DV) dv[roff + cc] = from_f32<T>(acc[i][j]);
    }
  }
}

// ---------------------------------------------------------------------------
// host side: one launcher per phase (the plan in fbla_plan.hip strings them together)
// ---------------------------------------------------------------------------

// Tokens per reduction chunk: enough chunks to give every CU several workgroups,
// few enough that the partial buffer stays small.
int state_chunk(const Prob& p) {
  const int64_t nh = (int64_t)p.N * p.H;
  const int64_t target_wgs = 1024;
  int64_t chunk = cdiv64((int64_t)p.L * nh, target_wgs);
  chunk = cdiv64(chunk, kTile) * kTile;
  if (chunk < 2 * kTile) chunk = 2 * kTile;
  return (int)chunk;
}

static int micro(const Prob& p) {
  const int d = p.DK > p.DV ? p.DK : p.DV;
  return d <= 32 ? 2 : (d <= 64 ? 4 : 8);
}

template <typename T>
static void state_partial_t(const Prob& p, const void* kn, const void* v, const void* kd,
                            float* partial, int chunk, int nchunks, hipStream_t st) {
  const dim3 grid((unsigned)((int64_t)p.N * p.H * nchunks)), block(kThreads);
  const T *a = (const T*)kn, *b = (const T*)v, *c = (const T*)kd;
  switch (micro(p)) {
    case 2: state_partial_kernel<T, 2><<<grid, block, 0, st>>>(p, a, b, c, partial, chunk, nchunks); break;
    case 4: state_partial_kernel<T, 4><<<grid, block, 0, st>>>(p, a, b, c, partial, chunk, nchunks); break;
    default: state_partial_kernel<T, 8><<<grid, block, 0, st>>>(p, a, b, c, partial, chunk, nchunks); break;
  }
}

void state_partial(const Prob& p, int dtype, const void* kn, const void* v, const void* kd,
                   float* partial, int chunk, int nchunks, hipStream_t st) {
  if (dtype == kF16) state_partial_t<_Float16>(p, kn, v, kd, partial, chunk, nchunks, st);
  else if (dtype == kBF16) state_partial_t<__bf16>(p, kn, v, kd, partial, chunk, nchunks, st);
  else state_partial_t<float>(p, kn, v, kd, partial, chunk, nchunks, st);
}

// The same with four consecutive elements per thread (16-byte loads and stores): head dims that
// are multiples of four.  A quarter of the workgroups: with thousands of (sequence, head) pairs the
// kernel's time is the time to start its workgroups.
__global__ __launch_bounds__(kThreads) void state_reduce4_kernel(
    Prob p, const float* __restrict__ partial, int chunk, int nchunks, float* __restrict__ mat,
    float* __restrict__ mat_t, float* __restrict__ vec, int blocks_per_head) {
  typedef float f32x4 __attribute__((ext_vector_type(4)));
  const int nh = blockIdx.x / blocks_per_head, blk = blockIdx.x - nh * blocks_per_head;
  const int n = nh / p.H;
  int64_t bos;
  int len;
  seq_range(p, n, bos, len);
  const int DK = p.DK, DV = p.DV, E = DK * DV, stride = E + DK;
  const int e = 4 * (blk * kThreads + threadIdx.x);
  if (e >= stride) return;
  const int nvalid = len > 0 ? min(nchunks, (len + chunk - 1) / chunk) : 0;
  const float* src = partial + partial_slot(p, n, nh - n * p.H, 0, nchunks) * stride + e;
  const int64_t cstride = (int64_t)stride * partial_step(p);
  f32x4 a = {0.f, 0.f, 0.f, 0.f};
  int c = 0;
  for (; c + 4 <= nvalid; c += 4) {  // fixed order: chunk 0, 1, 2, ...
    const f32x4 x0 = *reinterpret_cast<const f32x4*>(src + c * cstride);
    const f32x4 x1 = *reinterpret_cast<const f32x4*>(src + (c + 1) * cstride);
    const f32x4 x2 = *reinterpret_cast<const f32x4*>(src + (c + 2) * cstride);
    const f32x4 x3 = *reinterpret_cast<const f32x4*>(src + (c + 3) * cstride);
    a = (((a + x0) + x1) + x2) + x3;
  }
  for (; c < nvalid; ++c) a += *reinterpret_cast<const f32x4*>(src + c * cstride);
  if (e < E) {
    a *= seq_scale(p, len);
    *reinterpret_cast<f32x4*>(mat + (int64_t)nh * E + e) = a;
    if (mat_t) {
      const int dk = e / DV, dv = e - dk * DV;  // four consecutive dv of one dk
#pragma unroll
      for (int i = 0; i < 4; ++i) mat_t[(int64_t)nh * E + (dv + i) * DK + dk] = a[i];
    }
  } else if (vec) {
    const f32x4 r = {len > 0 ? a[0] / (float)len : 0.f, len > 0 ? a[1] / (float)len : 0.f,
                     len > 0 ? a[2] / (float)len : 0.f, len > 0 ? a[3] / (float)len : 0.f};
    *reinterpret_cast<f32x4*>(vec + (int64_t)nh * DK + (e - E)) = r;
  }
}

void state_reduce(const Prob& p, const float* partial, int chunk, int nchunks, float* mat,
                  float* mat_t, float* vec, hipStream_t st) {
  if (p.DK % 4 == 0 && p.DV % 4 == 0) {
    const int blocks_per_head = (p.DK * p.DV + p.DK + 4 * kThreads - 1) / (4 * kThreads);
    state_reduce4_kernel<<<dim3((unsigned)((int64_t)p.N * p.H * blocks_per_head)), dim3(kThreads), 0, st>>>(
        p, partial, chunk, nchunks, mat, mat_t, vec, blocks_per_head);
    return;
  }
  const int blocks_per_head = (p.DK * p.DV + p.DK + kThreads - 1) / kThreads;
  state_reduce_kernel<<<dim3((unsigned)((int64_t)p.N * p.H * blocks_per_head)), dim3(kThreads), 0, st>>>(
      p, partial, chunk, nchunks, mat, mat_t, vec, blocks_per_head);
}

// count matrices [rs][cs] -> [rd][cd]: the common part copied, the rest of the destination zero (widening
// token rows to the next row length the matrix-core kernels take, and narrowing their results back).
// Consecutive threads take consecutive destination elements.
template <typename E>
__global__ __launch_bounds__(kThreads) void resize_matrices_kernel(const E* __restrict__ src, int64_t rs, int cs,
                                                                   E* __restrict__ dst, int64_t rd, int cd,
                                                                   int64_t total) {
  for (int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x; i < total; i += (int64_t)gridDim.x * kThreads) {
    const int64_t row_all = i / cd;
    const int c = (int)(i - row_all * cd);
    const int64_t m = row_all / rd, r = row_all - m * rd;
    dst[i] = (r < rs && c < cs) ? src[(m * rs + r) * cs + c] : E(0);
  }
}
// The same for one matrix of many rows whose number does not change (token tensors): every workgroup takes a
// span of kResizeSpan consecutive destination elements, thread t the elements t, t + 256, ... of it (whole
// 128-byte pieces per wave instruction), with one division per thread and the row / column carried along.
constexpr int kResizePer = 16, kResizeSpan = kThreads * kResizePer;
template <typename E>
__global__ __launch_bounds__(kThreads) void resize_rows_kernel(const E* __restrict__ src, int cs, E* __restrict__ dst,
                                                               int cd, int64_t total) {
  const int64_t base = (int64_t)blockIdx.x * kResizeSpan;
  const int64_t row0 = base / cd;  // (uniform: scalar arithmetic)
  const uint32_t c0 = (uint32_t)(base - row0 * cd) + threadIdx.x;
  uint32_t rowd = c0 / (uint32_t)cd, c = c0 - rowd * (uint32_t)cd;
  const uint32_t left = (uint32_t)(total - base < kResizeSpan ? total - base : kResizeSpan);
  const E* s = src + row0 * cs;
  E* d = dst + base;
  E val[kResizePer];
#pragma unroll
  for (int u = 0; u < kResizePer; ++u) {
    const uint32_t off = threadIdx.x + u * kThreads;
    const bool in = off < left && c < (uint32_t)cs;
    val[u] = __builtin_nontemporal_load(s + (in ? (size_t)rowd * cs + c : 0));  // read once: streaming hint
    val[u] = in ? val[u] : E(0);
    c += kThreads;
    while (c >= (uint32_t)cd) {
      c -= cd;
      ++rowd;
    }
  }
#pragma unroll
  for (int u = 0; u < kResizePer; ++u) {
    const uint32_t off = threadIdx.x + u * kThreads;
    if (off < left) d[off] = val[u];
  }
}

void resize_matrices(const void* src, int64_t rs, int cs, void* dst, int64_t rd, int cd, int64_t count, int elem_bytes,
                     hipStream_t st) {
  const int64_t total = count * rd * cd;
  if (total <= 0) return;
  if (count == 1 && rs == rd) {
    // rows of a whole number of 8-byte pieces on both sides move as such (a quarter / half of the
    // load and store instructions)
    const int per8 = 8 / elem_bytes;
    if (cs % per8 == 0 && cd % per8 == 0 && (reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) % 8 == 0) {
      const unsigned spans8 = (unsigned)cdiv64(total / per8, kResizeSpan);
      resize_rows_kernel<uint64_t><<<dim3(spans8), dim3(kThreads), 0, st>>>((const uint64_t*)src, cs / per8, (uint64_t*)dst,
                                                                           cd / per8, total / per8);
      return;
    }
    const unsigned spans = (unsigned)cdiv64(total, kResizeSpan);
    if (elem_bytes == 2)
      resize_rows_kernel<uint16_t><<<dim3(spans), dim3(kThreads), 0, st>>>((const uint16_t*)src, cs, (uint16_t*)dst, cd,
                                                                          total);
    else
      resize_rows_kernel<uint32_t><<<dim3(spans), dim3(kThreads), 0, st>>>((const uint32_t*)src, cs, (uint32_t*)dst, cd,
                                                                          total);
    return;
  }
  const unsigned grid = (unsigned)std::min<int64_t>(cdiv64(total, kThreads), 1 << 20);
  if (elem_bytes == 2)
    resize_matrices_kernel<uint16_t><<<dim3(grid), dim3(kThreads), 0, st>>>((const uint16_t*)src, rs, cs, (uint16_t*)dst,
                                                                           rd, cd, total);
  else
    resize_matrices_kernel<uint32_t><<<dim3(grid), dim3(kThreads), 0, st>>>((const uint32_t*)src, rs, cs, (uint32_t*)dst,
                                                                           rd, cd, total);
}

// Two queries sharing keys and values: the state's value columns [0, DV/2) serve the first query,
// [DV/2, DV) the second.  split: lo[nh][r][c] = mat[nh][r][c], hi[nh][r][c] = mat[nh][r][DV/2 + c];
// join is the inverse for the matrices and adds the two vectors.
__global__ __launch_bounds__(kThreads) void split_columns_kernel(const float* __restrict__ mat,
                                                                 float* __restrict__ lo, float* __restrict__ hi,
                                                                 int DK, int DV) {
  const int half = DV / 2;
  const int64_t base = (int64_t)blockIdx.x * DK * DV, hbase = (int64_t)blockIdx.x * DK * half;
  for (int e = threadIdx.x; e < DK * DV; e += kThreads) {
    const int r = e / DV, c = e - r * DV;
    if (c < half) lo[hbase + r * half + c] = mat[base + e];
    else hi[hbase + r * half + c - half] = mat[base + e];
  }
}
__global__ __launch_bounds__(kThreads) void join_columns_kernel(
    const float* __restrict__ lo, const float* __restrict__ hi, const float* __restrict__ vec_lo,
    const float* __restrict__ vec_hi, float* __restrict__ mat, float* __restrict__ vec, int DK, int DV) {
  const int half = DV / 2;
  const int64_t base = (int64_t)blockIdx.x * DK * DV, hbase = (int64_t)blockIdx.x * DK * half;
  for (int e = threadIdx.x; e < DK * DV; e += kThreads) {
    const int r = e / DV, c = e - r * DV;
    mat[base + e] = c < half ? lo[hbase + r * half + c] : hi[hbase + r * half + c - half];
  }
  if (vec)
    for (int e = threadIdx.x; e < DK; e += kThreads)
      vec[(int64_t)blockIdx.x * DK + e] = vec_lo[(int64_t)blockIdx.x * DK + e] + vec_hi[(int64_t)blockIdx.x * DK + e];
}
void split_columns(const Prob& p, const float* mat, float* lo, float* hi, hipStream_t st) {
  split_columns_kernel<<<dim3((unsigned)((int64_t)p.N * p.H)), dim3(kThreads), 0, st>>>(mat, lo, hi, p.DK, p.DV);
}
void join_columns(const Prob& p, const float* lo, const float* hi, const float* vec_lo, const float* vec_hi,
                  float* mat, float* vec, hipStream_t st) {
  join_columns_kernel<<<dim3((unsigned)((int64_t)p.N * p.H)), dim3(kThreads), 0, st>>>(lo, hi, vec_lo, vec_hi, mat,
                                                                                       vec, p.DK, p.DV);
}

void transpose_state(const Prob& p, const float* mat, float* mat_t, hipStream_t st) {
  transpose_state_kernel<<<dim3((unsigned)((int64_t)p.N * p.H)), dim3(kThreads), 0, st>>>(
      mat, mat_t, p.DK, p.DV);
}

template <typename T>
static void output_t(const Prob& p, const void* qn, const void* qd, const float* S, const float* km,
                     void* o, hipStream_t st) {
  const int ntiles = (int)cdiv64(p.L, kTile);
  output_kernel<T><<<dim3((unsigned)((int64_t)p.N * p.H * ntiles)), dim3(kThreads), 0, st>>>(
      p, (const T*)qn, (const T*)qd, S, km, (T*)o, ntiles);
}

void output(const Prob& p, int dtype, const void* qn, const void* qd, const float* S,
            const float* km, void* o, hipStream_t st) {
  if (dtype == kF16) output_t<_Float16>(p, qn, qd, S, km, o, st);
  else if (dtype == kBF16) output_t<__bf16>(p, qn, qd, S, km, o, st);
  else output_t<float>(p, qn, qd, S, km, o, st);
}

template <typename T>
static void bwd_a_t(const Prob& p, const void* qn, const void* qd, const void* dout, const float* S,
                    const float* St, const float* km, void* dqn, void* dqd, float* partial,
                    int chunk, int nchunks, hipStream_t st) {
  const dim3 grid((unsigned)((int64_t)p.N * p.H * nchunks)), block(kThreads);
  const T *a = (const T*)qn, *b = (const T*)qd, *c = (const T*)dout;
  T *x = (T*)dqn, *y = (T*)dqd;
  switch (micro(p)) {
    case 2: bwd_a_kernel<T, 2><<<grid, block, 0, st>>>(p, a, b, c, S, St, km, x, y, partial, chunk, nchunks); break;
    case 4: bwd_a_kernel<T, 4><<<grid, block, 0, st>>>(p, a, b, c, S, St, km, x, y, partial, chunk, nchunks); break;
    default: bwd_a_kernel<T, 8><<<grid, block, 0, st>>>(p, a, b, c, S, St, km, x, y, partial, chunk, nchunks); break;
  }
}

void bwd_a(const Prob& p, int dtype, const void* qn, const void* qd, const void* dout,
           const float* S, const float* St, const float* km, void* dqn, void* dqd, float* partial,
           int chunk, int nchunks, hipStream_t st) {
  if (dtype == kF16) bwd_a_t<_Float16>(p, qn, qd, dout, S, St, km, dqn, dqd, partial, chunk, nchunks, st);
  else if (dtype == kBF16) bwd_a_t<__bf16>(p, qn, qd, dout, S, St, km, dqn, dqd, partial, chunk, nchunks, st);
  else bwd_a_t<float>(p, qn, qd, dout, S, St, km, dqn, dqd, partial, chunk, nchunks, st);
}

template <typename T>
static void bwd_b_t(const Prob& p, const void* kn, const void* v, const float* dS, const float* dSt,
                    const float* dkm, void* dkn, void* dkd, void* dv, float dkm_scale, hipStream_t st) {
  const int ntiles = (int)cdiv64(p.L, kTile);
  bwd_b_kernel<T><<<dim3((unsigned)((int64_t)p.N * p.H * ntiles)), dim3(kThreads), 0, st>>>(
      p, (const T*)kn, (const T*)v, dS, dSt, dkm, (T*)dkn, (T*)dkd, (T*)dv, ntiles, dkm_scale);
}

void bwd_b(const Prob& p, int dtype, const void* kn, const void* v, const float* dS,
           const float* dSt, const float* dkm, void* dkn, void* dkd, void* dv, hipStream_t st,
           float dkm_scale) {
  if (dtype == kF16) bwd_b_t<_Float16>(p, kn, v, dS, dSt, dkm, dkn, dkd, dv, dkm_scale, st);
  else if (dtype == kBF16) bwd_b_t<__bf16>(p, kn, v, dS, dSt, dkm, dkn, dkd, dv, dkm_scale, st);
  else bwd_b_t<float>(p, kn, v, dS, dSt, dkm, dkn, dkd, dv, dkm_scale, st);
}

template <typename T>
__global__ __launch_bounds__(kThreads) void broadcast_rows_kernel(Prob p, const float* __restrict__ vec,
                                                                  T* __restrict__ out, int ntiles, float factor) {
  const int nh = blockIdx.x / ntiles, tile = blockIdx.x - nh * ntiles;
  const int n = nh / p.H, h = nh - n * p.H;
  int64_t bos, row0, rstride;
  int len;
  seq_range(p, n, bos, len);
  const int t0 = tile * kTile;
  if (t0 >= len) return;
  const int nvalid = min(kTile, len - t0);
  row_base(p, n, h, bos, row0, rstride);
  const int DK = p.DK;
  for (int i = threadIdx.x; i < nvalid * DK; i += kThreads) {
    const int t = i / DK, d = i - t * DK;
    out[(row0 + (int64_t)(t0 + t) * rstride) * DK + d] = from_f32<T>(vec[(int64_t)nh * DK + d] * factor);
  }
}

// The same for rows made of a power-of-two number of 16-byte pieces: a thread builds its piece of the
// row once and stores it (streaming) to that piece of every row it owns.
constexpr int kBroadcastRows = 256;
template <typename T>
__global__ __launch_bounds__(kThreads) void broadcast_rows16_kernel(Prob p, const float* __restrict__ vec,
                                                                    T* __restrict__ out, int nchunks,
                                                                    float factor, int piece_shift) {
  typedef uint32_t words4 __attribute__((ext_vector_type(4)));
  constexpr int E = 16 / (int)sizeof(T);
  const int nh = blockIdx.x / nchunks, chunk = blockIdx.x - nh * nchunks;
  const int n = nh / p.H, h = nh - n * p.H;
  int64_t bos, row0, rstride;
  int len;
  seq_range(p, n, bos, len);
  const int t0 = chunk * kBroadcastRows;
  if (t0 >= len) return;
  const int nvalid = min(kBroadcastRows, len - t0);
  row_base(p, n, h, bos, row0, rstride);
  const int piece = threadIdx.x & ((1 << piece_shift) - 1), first = threadIdx.x >> piece_shift;
  const int step = kThreads >> piece_shift;
  union { T e[E]; words4 w; } val;
  for (int i = 0; i < E; ++i) val.e[i] = from_f32<T>(vec[(int64_t)nh * p.DK + piece * E + i] * factor);
  T* dst = out + (row0 + (int64_t)(t0 + first) * rstride) * p.DK + piece * E;
  const int64_t stride = (int64_t)step * rstride * p.DK;
  for (int t = first; t < nvalid; t += step, dst += stride) __builtin_nontemporal_store(val.w, (words4*)dst);
}

template <typename T>
static bool broadcast_rows16(const Prob& p, const float* vec, T* out, hipStream_t st, float factor) {
  const int row_bytes = p.DK * (int)sizeof(T), pieces = row_bytes / 16;
  if (row_bytes % 16 || (pieces & (pieces - 1)) || pieces > kThreads || ((uintptr_t)out & 15)) return false;
  int shift = 0;
  while ((1 << shift) < pieces) ++shift;
  const int nchunks = (int)cdiv64(p.L, kBroadcastRows);
  broadcast_rows16_kernel<T><<<dim3((unsigned)((int64_t)p.N * p.H * nchunks)), dim3(kThreads), 0, st>>>(
      p, vec, out, nchunks, factor, shift);
  return true;
}

// every row of out ([.., DK]) = vec of its (sequence, head): dk of the decoupled operator
void broadcast_rows(const Prob& p, int dtype, const float* vec, void* out, hipStream_t st, float factor) {
  if (dtype == kF16 ? broadcast_rows16(p, vec, (_Float16*)out, st, factor)
      : dtype == kBF16 ? broadcast_rows16(p, vec, (__bf16*)out, st, factor)
                       : broadcast_rows16(p, vec, (float*)out, st, factor))
    return;
  const int ntiles = (int)cdiv64(p.L, kTile);
  const dim3 grid((unsigned)((int64_t)p.N * p.H * ntiles)), block(kThreads);
  if (dtype == kF16) broadcast_rows_kernel<_Float16><<<grid, block, 0, st>>>(p, vec, (_Float16*)out, ntiles, factor);
  else if (dtype == kBF16) broadcast_rows_kernel<__bf16><<<grid, block, 0, st>>>(p, vec, (__bf16*)out, ntiles, factor);
  else broadcast_rows_kernel<float><<<grid, block, 0, st>>>(p, vec, (float*)out, ntiles, factor);
}

// One thread per sequence j counts the sequences that come before it in the order (longer,
// or as long with a smaller index); the lengths pass through LDS in tiles of the block size.
__global__ __launch_bounds__(256) void rank_sequences_kernel(const int32_t* __restrict__ cu, int N,
                                                             int32_t* __restrict__ perm) {
  __shared__ int tile[256];
  const int j = blockIdx.x * 256 + threadIdx.x;
  const int lj = j < N ? cu[j + 1] - cu[j] : 0;
  int r = 0;
  for (int base = 0; base < N; base += 256) {
    const int i = base + threadIdx.x;
    tile[threadIdx.x] = i < N ? cu[i + 1] - cu[i] : -1;
    __syncthreads();
    const int cnt = min(256, N - base);
    for (int t = 0; t < cnt; ++t) {
      const int li = tile[t];
      r += (li > lj) || (li == lj && base + t < j);
    }
    __syncthreads();
  }
  if (j < N) perm[r] = j;
}

// base[n] = number of chunks of `chunk` tokens of the sequences before n, base[N] = all of them.
// One workgroup walks the sequences 256 at a time with a running total.
__global__ __launch_bounds__(256) void chunk_bases_kernel(const int32_t* __restrict__ cu, int N, int chunk,
                                                         int32_t* __restrict__ base) {
  __shared__ int scan[256];
  int total = 0;
  for (int first = 0; first < N; first += 256) {
    const int j = first + threadIdx.x;
    const int len = j < N ? cu[j + 1] - cu[j] : 0;
    const int cnt = len > 0 ? (len + chunk - 1) / chunk : 0;
    scan[threadIdx.x] = cnt;
    __syncthreads();
    for (int off = 1; off < 256; off <<= 1) {  // inclusive scan
      const int add = threadIdx.x >= off ? scan[threadIdx.x - off] : 0;
      __syncthreads();
      scan[threadIdx.x] += add;
      __syncthreads();
    }
    if (j < N) base[j] = total + scan[threadIdx.x] - cnt;
    total += scan[255];
    __syncthreads();
  }
  if (threadIdx.x == 0) base[N] = total;
}

void chunk_bases(const Prob& p, int chunk, int32_t* base, hipStream_t st) {
  chunk_bases_kernel<<<dim3(1), dim3(256), 0, st>>>(p.cu, p.N, chunk, base);
}

void rank_sequences(const Prob& p, int32_t* perm, hipStream_t st) {
  rank_sequences_kernel<<<dim3((unsigned)((p.N + 255) / 256)), dim3(256), 0, st>>>(p.cu, p.N, perm);
}

}  // namespace generic
}  // namespace fbla
