// Shared host/device definitions for the gfx950 bidirectional linear-attention kernels.
//
// Terminology (follows flash_bla): a *sequence* is one (batch) entry of a dense
// [B,H,L,D] tensor or one [cu[i],cu[i+1]) range of a packed [T,H,D] tensor; the
// *state* of a (sequence, head) is S = scale * K^T V (DK x DV, fp32) together
// with km = mean_t k_t (DK, fp32).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdlib.h>

namespace fbla {

enum DType : int { kF16 = 0, kBF16 = 1, kF32 = 2 };

enum Flags : int {
  kNormalize = 1,     // divide by z = q.km + eps (linear_attn); off = simple_la
  kDecoupled = 2,     // numerator uses q_rope/k_rope, denominator q/k
  kDefaultScale = 4,  // varlen only: scale = 1/len_i per sequence
  kElu1 = 8,          // forward only: q and k arrive before the feature map, the kernels apply elu(x) + 1 on load
  kElu1Grad = 16,     // backward only: q and k are the mapped tensors phi(x) = elu(x) + 1 and dq, dk are wanted
                      // with respect to x: the kernels multiply them by phi'(x) = min(phi(x), 1)
  kXcdOrder = 256,    // internal (set per launch): packed batches keep a sequence's heads on one XCD
  kInterleave = 512,  // internal (set per launch): the workgroups of a head take interleaved token steps
};
// what a caller may pass; the per-launch bits are the plan's alone (set from outside they would change
// how the kernels walk without changing how the partials are counted)
constexpr int kPublicFlags = kNormalize | kDecoupled | kDefaultScale | kElu1 | kElu1Grad;

// One problem instance.  Dense: cu == nullptr, N = batch, every sequence has L
// tokens and tensors are [N,H,L,D].  Packed: cu = int32[N+1] on the device and
// tensors are [T_total,H,D].
// Packed batches are walked longest sequence first.  Up to kRankInline sequences every
// workgroup ranks the lengths itself (in LDS, a fraction of a microsecond); up to kRankMax a
// small kernel writes the order once per call (Prob::perm); beyond that the order is the
// index order.
constexpr int kRankInline = 128;
constexpr int kRankMax = 1 << 16;

struct Prob {
  const int32_t* cu;
  const int32_t* perm;  // packed: perm[r] = index of the sequence with the r-th largest length, or null
  const int32_t* chunk_base;  // packed, skewed batches: chunk_base[n] = number of reduction chunks of the
                              // sequences before n (one partial per chunk that exists), or null: every
                              // (sequence, head) has room for the chunks of the longest sequence
  int N, H, L;  // L: dense length, or max_seqlen upper bound when packed
  int Lk;       // dense only: number of key / value tokens when it differs from L (the number of
                // queries), else 0.  Only the plan looks at it: kernels get a problem whose L is
                // the length of the side they walk.
  int64_t T;    // total tokens (dense: N*L)
  int DK, DV;
  float scale;
  float eps;
  int flags;
};

// The reduction kernels (forward state, backward pass A) write one partial per chunk of a
// (sequence, head); their consumers add them up in chunk order.  Slot of the partial of chunk c
// (of nchunks provided for) of (sequence n, head h), and the distance in slots between the
// partials of consecutive chunks.
__device__ __forceinline__ int64_t partial_slot(const Prob& p, int n, int h, int c, int nchunks) {
  return p.chunk_base ? ((int64_t)p.chunk_base[n] + c) * p.H + h : ((int64_t)n * p.H + h) * nchunks + c;
}
__device__ __forceinline__ int64_t partial_step(const Prob& p) { return p.chunk_base ? p.H : 1; }

// Token range of sequence n.
__device__ __forceinline__ void seq_range(const Prob& p, int n, int64_t& bos, int& len) {
  if (p.cu) {
    int b = p.cu[n];
    bos = b;
    len = p.cu[n + 1] - b;
  } else {
    bos = 0;
    len = p.L;
  }
}

// Row index (units of D-element rows) of local token 0 of (n,h) and the row
// stride between consecutive tokens.
__device__ __forceinline__ void row_base(const Prob& p, int n, int h, int64_t bos,
                                         int64_t& row0, int64_t& rstride) {
  if (p.cu) {
    row0 = bos * p.H + h;
    rstride = p.H;
  } else {
    row0 = ((int64_t)n * p.H + h) * p.L;
    rstride = 1;
  }
}

__device__ __forceinline__ float seq_scale(const Prob& p, int len) {
  return (p.flags & kDefaultScale) ? (len > 0 ? 1.0f / (float)len : 0.0f) : p.scale;
}

template <typename T> __device__ __forceinline__ float to_f32(T x) { return (float)x; }
template <typename T> __device__ __forceinline__ T from_f32(float x) { return (T)x; }

// Integer launch-geometry constants.  A build with -DFBLA_TUNING (make TUNING=1, for sweeps and A/B
// runs) lets the environment variable `name` replace the default; the shipped library ignores the
// environment: the kernels' alignment assumptions are only tested with the defaults.
inline int tuning_knob(const char* name, int dflt, bool zero_ok = false) {
#ifdef FBLA_TUNING
  const char* v = getenv(name);
  if (v && (atoi(v) > 0 || (zero_ok && v[0] == '0'))) return atoi(v);
#else
  (void)name;
  (void)zero_ok;
#endif
  return dflt;
}

inline int64_t cdiv64(int64_t a, int64_t b) { return (a + b - 1) / b; }
inline size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

// Error reporting across the C ABI (thread-local message, integer codes).
void set_error(const char* fmt, ...);

enum Err : int {
  kOk = 0,
  kErrBadArg = -1,
  kErrUnsupported = -2,
  kErrWorkspace = -3,
  kErrLaunch = -4,
};

}  // namespace fbla
