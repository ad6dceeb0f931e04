// The plan: which kernels run, in which order, for each entry point, and how the
// caller's workspace is carved up.  MFMA kernels are used for the shapes they
// cover (16-bit inputs with head dims that are multiples of 8 up to 128, fp32 inputs with head dims
// that are multiples of 4 up to 128, up to 64 for the decoupled operator); other head dims run on
// them through zero-widened copies, what is left runs on the generic kernels.
//
// forward :  state partials -> fixed-order reduce (S, km) -> output rows
// backward:  S^T -> pass A (dq, partial dS/dkm) -> reduce (s dS, its transpose, dkm/L)
//            -> pass B (dk, dv)
//
// A dense problem may have fewer (or more) keys than queries (Prob::Lk): the state kernel and
// pass B then walk the Lk key / value tokens, the output kernel and pass A the L query tokens,
// each with a problem of its own length.  The reductions stay separate kernels (or direct
// stores) in that case, and dkm, which pass A leaves divided by the number of queries, is
// rescaled to dkm / Lk where pass B adds it.  MFMA path only.
#include <stdlib.h>

#include "fbla_kernels.h"

namespace fbla {
namespace plan {

// true when keys and queries differ in number
static bool cross(const Prob& p) { return !p.cu && p.Lk > 0 && p.Lk != p.L; }
// the problem as the kernels of one side see it
static Prob query_side(const Prob& p) {
  Prob s = p;
  s.Lk = 0;
  return s;
}
static Prob key_side(const Prob& p) {
  Prob s = p;
  if (cross(p)) {
    s.L = p.Lk;
    s.T = (int64_t)p.N * p.Lk;
  }
  s.Lk = 0;
  return s;
}

static size_t state_bytes(const Prob& p) {
  return align_up((size_t)p.N * p.H * p.DK * p.DV * sizeof(float), 256);
}
static size_t vec_bytes(const Prob& p) {
  return align_up((size_t)p.N * p.H * p.DK * sizeof(float), 256);
}
// Packed batches whose longest sequence has many more chunks than the others (one long sequence
// among short ones): the partials get one slot per chunk that exists instead of the longest
// sequence's number of chunks for every (sequence, head).  The sequences have at most
// T / chunk + N chunks together whatever their lengths are, which bounds the storage on the host;
// a one-workgroup kernel writes each sequence's first slot (Prob::chunk_base) once per call.
// Only where every kernel that touches the partials knows that layout: the 16-bit matrix-core path.
static bool compact_partials(const Prob& p, int dtype, int chunk) {
  if (!p.cu || dtype == kF32 || !mfma::supported(p, dtype)) return false;
  const int64_t nchunks = cdiv64(p.L, chunk);
  return nchunks >= 4 && (int64_t)p.N * nchunks > 2 * (cdiv64(p.T, chunk) + p.N);
}
static size_t chunk_base_bytes(const Prob& p) { return align_up((size_t)(p.N + 1) * sizeof(int32_t), 256); }
// partials (| first slot of every sequence)
static size_t partial_bytes(const Prob& p, int dtype, int chunk) {
  const size_t slot = ((size_t)p.DK * p.DV + p.DK) * sizeof(float);
  if (compact_partials(p, dtype, chunk))
    return align_up((size_t)(cdiv64(p.T, chunk) + p.N) * p.H * slot, 256) + chunk_base_bytes(p);
  const int64_t nchunks = cdiv64(p.L, chunk);
  return align_up((size_t)p.N * p.H * nchunks * slot, 256);
}
// The problem with its chunk bases, written behind the partials at the start of `workspace`.
static Prob with_chunk_bases(const Prob& p, int dtype, int chunk, void* workspace, hipStream_t st) {
  Prob r = p;
  if (compact_partials(p, dtype, chunk)) {
    int32_t* base = reinterpret_cast<int32_t*>((char*)workspace + partial_bytes(p, dtype, chunk) - chunk_base_bytes(p));
    generic::chunk_bases(p, chunk, base, st);
    r.chunk_base = base;
  }
  return r;
}
static int fwd_chunk(const Prob& p, int dtype) {
  return mfma::supported(p, dtype) ? mfma::state_chunk(p) : generic::state_chunk(p);
}
static int bwd_chunk(const Prob& p, int dtype) {
  if (mfma::bwd_a_supported(p, dtype)) return mfma::bwd_a_chunk(p);
  return mfma::supported(p, dtype) ? mfma::state_chunk(p) : generic::state_chunk(p);
}
// per-row scalars 1/z_t and dz_t of the two-kernel backward pass A
static size_t tokscal_bytes(const Prob& p, int dtype) {
  if (!mfma::supported(p, dtype) || mfma::bwd_a_supported(p, dtype)) return 0;
  return align_up((size_t)2 * p.T * p.H * sizeof(float), 256);
}

// The rows kernels can sum the reduction partials in their prologue (saving the
// reduce launch) or read a matrix reduced by a separate kernel.  Every workgroup
// of a head repeats the sum, so folding pays only while that extra traffic is
// small next to the cost of one more dependent launch.
static bool fold_reduce(const Prob& p, int reduce_nchunks, int DR, int DC) {
  const int64_t rows_nchunks = cdiv64(p.L, mfma::rows_chunk(p, DR, DC));
  const double extra = (double)p.N * p.H * (double)(rows_nchunks - 1) * reduce_nchunks *
                       ((double)p.DK * p.DV + p.DK) * sizeof(float);
  static const double limit = tuning_knob("FBLA_FOLD_MAX_MB", 16) * 1e6;
  return extra <= limit;
}

// the walking order of a packed batch with too many sequences to rank inside every workgroup
static size_t perm_bytes(const Prob& p) {
  // (the in-workgroup ranking has LDS for kRankInline lengths)
  static const int inline_max = std::min(tuning_knob("FBLA_RANK_INLINE", kRankInline, true), kRankInline);
  return (p.cu && p.N > inline_max && p.N >= 2 && p.N <= kRankMax) ? align_up((size_t)p.N * sizeof(int32_t), 256) : 0;
}
// Writes the order behind the first `used` bytes of the workspace and returns the problem with it.
static Prob with_order(const Prob& p, void* workspace, size_t used, hipStream_t st) {
  Prob r = p;
  if (perm_bytes(p)) {
    int32_t* perm = reinterpret_cast<int32_t*>((char*)workspace + used);
    generic::rank_sequences(p, perm, st);
    r.perm = perm;
  }
  return r;
}

// ---- head dims between the row lengths the matrix-core kernels take --------------------------
// 16-bit rows are moved in 16-byte pieces (head dims that are multiples of 8), fp32 rows likewise
// (multiples of 4).  A problem with another head dim (17 x 13, 100 x 100: shapes of the reference's
// test matrix, tests/ops/test_varlen_linear_attn.py:15-18) is widened to the next such row length
// with zeros in workspace copies of its tensors, run on the matrix-core kernels, and its results are
// narrowed back: zero features add nothing to any sum of the operator, so the results are those of the
// original problem.  The copies cost two to three tensor passes per tensor; the shape-generic kernels
// they replace are five to ten times slower than the matrix-core ones.
static int elem_bytes(int dtype) { return dtype == kF32 ? 4 : 2; }
static int widened_dim(int d, int dtype) {
  const int unit = dtype == kF32 ? 4 : 8;
  return (d + unit - 1) / unit * unit;
}
static Prob widened(const Prob& p, int dtype) {
  Prob w = p;
  w.DK = widened_dim(p.DK, dtype);
  w.DV = widened_dim(p.DV, dtype);
  return w;
}
static bool widen(const Prob& p, int dtype) {
  if (mfma::supported(p, dtype)) return false;
  const Prob w = widened(p, dtype);
  return w.DK <= 128 && w.DV <= 128 && mfma::supported(w, dtype);
}
// rows of the tensors on the query side / on the key side
static int64_t query_rows(const Prob& p) { return p.cu ? p.T * p.H : (int64_t)p.N * p.H * p.L; }
static int64_t key_rows(const Prob& p) { return p.cu ? p.T * p.H : (int64_t)p.N * p.H * (cross(p) ? p.Lk : p.L); }
static size_t rows_bytes(int64_t rows, int d, int dtype) { return align_up((size_t)rows * d * elem_bytes(dtype), 256); }
// carves `bytes` out of the workspace
static void* take(char*& ws, size_t bytes) {
  void* r = ws;
  ws += bytes;
  return r;
}
// a widened copy of a token tensor (null stays null)
static const void* widen_rows(const void* src, int64_t rows, int d, int dw, int dtype, char*& ws, hipStream_t st) {
  if (!src) return nullptr;
  void* dst = take(ws, rows_bytes(rows, dw, dtype));
  generic::resize_matrices(src, rows, d, dst, rows, dw, 1, elem_bytes(dtype), st);
  return dst;
}

static size_t widened_fwd_bytes(const Prob& p, int dtype) {
  const Prob w = widened(p, dtype);
  const bool dec = p.flags & kDecoupled;
  return (dec ? 2 : 1) * (rows_bytes(query_rows(p), w.DK, dtype) + rows_bytes(key_rows(p), w.DK, dtype)) +
         rows_bytes(key_rows(p), w.DV, dtype) + rows_bytes(query_rows(p), w.DV, dtype) + state_bytes(w) + vec_bytes(w) +
         fwd_workspace_bytes(w, dtype);
}
static size_t widened_bwd_bytes(const Prob& p, int dtype) {
  const Prob w = widened(p, dtype);
  const bool dec = p.flags & kDecoupled;
  // inputs q, k, v, dO (+ rotary rows), gradients dq, dk, dv (+ rotary), state, mean key
  return (dec ? 4 : 2) * (rows_bytes(query_rows(p), w.DK, dtype) + rows_bytes(key_rows(p), w.DK, dtype)) +
         2 * rows_bytes(key_rows(p), w.DV, dtype) + rows_bytes(query_rows(p), w.DV, dtype) + state_bytes(w) +
         vec_bytes(w) + bwd_workspace_bytes(w, dtype);
}

static size_t fwd_used_bytes(const Prob& pc, int dtype) {
  const Prob p = key_side(pc);
  return partial_bytes(p, dtype, fwd_chunk(p, dtype));
}
static size_t bwd_used_bytes(const Prob& pc, int dtype) {
  const Prob p = query_side(pc);
  return partial_bytes(p, dtype, bwd_chunk(p, dtype)) + 3 * state_bytes(p) + vec_bytes(p) +
         tokscal_bytes(p, dtype);
}

// partials | walking order
size_t fwd_workspace_bytes(const Prob& pc, int dtype) {
  if (widen(pc, dtype)) return widened_fwd_bytes(pc, dtype);
  return fwd_used_bytes(pc, dtype) + perm_bytes(pc);
}

// partials | S^T | s*dS | (s*dS)^T | dkm/L | per-row scalars | walking order
size_t bwd_workspace_bytes(const Prob& pc, int dtype) {
  if (widen(pc, dtype)) return widened_bwd_bytes(pc, dtype);
  return bwd_used_bytes(pc, dtype) + perm_bytes(pc);
}

// Different numbers of queries and keys work for every operator family (the decoupled one too:
// its rotary and plain rows come in pairs of equal length on either side).
static int check_cross(const Prob&, int) { return kOk; }

static int widened_forward(const Prob& p, int dtype, const FwdArgs& a, hipStream_t st) {
  const Prob w = widened(p, dtype);
  const int64_t qr = query_rows(p), kr = key_rows(p), nh = (int64_t)p.N * p.H;
  char* ws = (char*)a.workspace;
  FwdArgs b = a;
  b.q = widen_rows(a.q, qr, p.DK, w.DK, dtype, ws, st);
  b.k = widen_rows(a.k, kr, p.DK, w.DK, dtype, ws, st);
  b.v = widen_rows(a.v, kr, p.DV, w.DV, dtype, ws, st);
  b.q_rope = widen_rows(a.q_rope, qr, p.DK, w.DK, dtype, ws, st);
  b.k_rope = widen_rows(a.k_rope, kr, p.DK, w.DK, dtype, ws, st);
  b.o = take(ws, rows_bytes(qr, w.DV, dtype));
  b.s = (float*)take(ws, state_bytes(w));
  b.km = (float*)take(ws, vec_bytes(w));
  b.workspace = ws;
  b.workspace_bytes = a.workspace_bytes - (size_t)(ws - (char*)a.workspace);
  int rc = forward(w, dtype, b, st);
  if (rc != kOk) return rc;
  generic::resize_matrices(b.o, qr, w.DV, a.o, qr, p.DV, 1, elem_bytes(dtype), st);
  generic::resize_matrices(b.s, w.DK, w.DV, a.s, p.DK, p.DV, nh, 4, st);
  if (a.km) generic::resize_matrices(b.km, 1, w.DK, a.km, 1, p.DK, nh, 4, st);
  return kOk;
}

static int widened_backward(const Prob& p, int dtype, const BwdArgs& a, hipStream_t st) {
  const Prob w = widened(p, dtype);
  const int64_t qr = query_rows(p), kr = key_rows(p), nh = (int64_t)p.N * p.H;
  const bool dec = p.flags & kDecoupled;
  char* ws = (char*)a.workspace;
  BwdArgs b = a;
  b.q = widen_rows(a.q, qr, p.DK, w.DK, dtype, ws, st);
  b.k = widen_rows(a.k, kr, p.DK, w.DK, dtype, ws, st);
  b.v = widen_rows(a.v, kr, p.DV, w.DV, dtype, ws, st);
  b.q_rope = widen_rows(a.q_rope, qr, p.DK, w.DK, dtype, ws, st);
  b.k_rope = widen_rows(a.k_rope, kr, p.DK, w.DK, dtype, ws, st);
  b.dout = widen_rows(a.dout, qr, p.DV, w.DV, dtype, ws, st);
  float* sw = (float*)take(ws, state_bytes(w));
  float* kmw = (float*)take(ws, vec_bytes(w));
  generic::resize_matrices(a.s, p.DK, p.DV, sw, w.DK, w.DV, nh, 4, st);
  if (a.km) generic::resize_matrices(a.km, 1, p.DK, kmw, 1, w.DK, nh, 4, st);
  b.s = sw;
  b.km = a.km ? kmw : nullptr;
  b.dq = take(ws, rows_bytes(qr, w.DK, dtype));
  b.dk = take(ws, rows_bytes(kr, w.DK, dtype));
  b.dv = take(ws, rows_bytes(kr, w.DV, dtype));
  b.dq_rope = dec ? take(ws, rows_bytes(qr, w.DK, dtype)) : nullptr;
  b.dk_rope = dec ? take(ws, rows_bytes(kr, w.DK, dtype)) : nullptr;
  b.workspace = ws;
  b.workspace_bytes = a.workspace_bytes - (size_t)(ws - (char*)a.workspace);
  int rc = backward(w, dtype, b, st);
  if (rc != kOk) return rc;
  const int eb = elem_bytes(dtype);
  generic::resize_matrices(b.dq, qr, w.DK, a.dq, qr, p.DK, 1, eb, st);
  generic::resize_matrices(b.dk, kr, w.DK, a.dk, kr, p.DK, 1, eb, st);
  generic::resize_matrices(b.dv, kr, w.DV, a.dv, kr, p.DV, 1, eb, st);
  if (dec) {
    generic::resize_matrices(b.dq_rope, qr, w.DK, a.dq_rope, qr, p.DK, 1, eb, st);
    generic::resize_matrices(b.dk_rope, kr, w.DK, a.dk_rope, kr, p.DK, 1, eb, st);
  }
  return kOk;
}

int forward(const Prob& pc_, int dtype, const FwdArgs& a, hipStream_t st) {
  int rc_cross = check_cross(pc_, dtype);
  if (rc_cross != kOk) return rc_cross;
  if (widen(pc_, dtype) && phase_mask() == kPhaseAll) return widened_forward(pc_, dtype, a, st);
  const Prob pc = with_order(pc_, a.workspace, fwd_used_bytes(pc_, dtype), st);
  const bool is_cross = cross(pc);
  const Prob p_ = key_side(pc);    // state kernel, reduce
  const Prob pq_ = query_side(pc);  // output kernel
  const bool dec = p_.flags & kDecoupled;
  const bool normalize = p_.flags & kNormalize;
  const void* qn = dec ? a.q_rope : a.q;
  const void* kn = dec ? a.k_rope : a.k;
  const bool fast = mfma::supported(p_, dtype);
  if (p_.flags & kElu1Grad) {
    set_error("FBLA_ELU1_GRAD is a flag of the backward entry points");
    return kErrBadArg;
  }
  if ((p_.flags & kElu1) && !(fast && dtype != kF32 && p_.DK == 64 && p_.DV == 64 && !dec)) {
    set_error("the feature map on load (FBLA_ELU1_QK) covers fp16 / bf16 heads of 64 x 64, not the decoupled operator");
    return kErrUnsupported;
  }
  const int chunk = fwd_chunk(p_, dtype);
  const int nchunks = (int)cdiv64(p_.L, chunk);
  float* partial = (float*)a.workspace;
  // (skewed packed batches: one partial per chunk that exists)
  const Prob p = with_chunk_bases(p_, dtype, chunk, a.workspace, st);
  Prob pq = pq_;
  pq.chunk_base = p.chunk_base;
  const unsigned phases = phase_mask();
  // one chunk per (sequence, head): the state kernel stores the finished S and km itself
  const bool direct = fast && nchunks == 1;
  if (phases & kPhaseFwdState) {
    if (fast)
      mfma::state(mfma::with_interleave(p, dtype, 1), dtype, kn, a.v, a.k, partial, chunk, nchunks, st,
                  direct ? a.s : nullptr, direct ? a.km : nullptr);
    else
      generic::state_partial(p, dtype, kn, a.v, a.k, partial, chunk, nchunks, st);
  }
  const bool fold = fast && !direct && !is_cross && dtype != kF32 && !mfma::pair_mode(p, dtype) &&
                    fold_reduce(p, nchunks, p.DK, p.DV);
  // tokens per partial as the consumers of the partials count them
  const int pchunk = fast ? mfma::partial_chunk(p, dtype, 1, chunk) : chunk;
  if (!fold && !direct && (phases & kPhaseFwdReduce))
    generic::state_reduce(p, partial, pchunk, nchunks, a.s, nullptr, a.km, st);
  if (phases & kPhaseFwdOutput) {
    if (fast) {
      mfma::RowsJob job{qn, normalize ? a.q : nullptr, a.s, p.DV, 1, a.km, nullptr, a.o};
      if (fold) {  // the output kernel sums the partials itself and stores S and km on the way
        job.mat = partial;
        job.pchunk = pchunk;
        job.pnchunks = nchunks;
        job.mat_out = a.s;
        job.vec_out = a.km;
      }
      int rc = mfma::rows(mfma::with_interleave(pq, dtype, 2), dtype, job, p.DK, p.DV, st);
      if (rc != kOk) return rc;
    } else {
      generic::output(pq, dtype, qn, a.q, a.s, a.km, a.o, st);
    }
  }
  return kOk;
}

int backward(const Prob& pc_, int dtype, const BwdArgs& a, hipStream_t st) {
  int rc_cross = check_cross(pc_, dtype);
  if (rc_cross != kOk) return rc_cross;
  if (widen(pc_, dtype) && phase_mask() == kPhaseAll) return widened_backward(pc_, dtype, a, st);
  if ((pc_.flags & kElu1) && !(pc_.flags & kElu1Grad)) {
    set_error("the feature map on load (FBLA_ELU1_QK) in a backward needs FBLA_ELU1_GRAD as well: dq, dk are then "
              "gradients with respect to the q, k given");
    return kErrUnsupported;
  }
  if ((pc_.flags & kElu1Grad) && !(dtype != kF32 && pc_.DK == 64 && pc_.DV == 64 && !(pc_.flags & kDecoupled) &&
                                   mfma::bwd_a_supported(pc_, dtype))) {
    set_error("gradients through the feature map (FBLA_ELU1_GRAD) cover fp16 / bf16 heads of 64 x 64, not the decoupled operator");
    return kErrUnsupported;
  }
  const Prob pc = with_order(pc_, a.workspace, bwd_used_bytes(pc_, dtype), st);
  const bool is_cross = cross(pc);
  const Prob p_ = query_side(pc);  // pass A, reduce
  const Prob pk_ = key_side(pc);   // pass B
  // (skewed packed batches: one partial per chunk that exists)
  const Prob p = with_chunk_bases(p_, dtype, bwd_chunk(p_, dtype), a.workspace, st);
  Prob pk = pk_;
  pk.chunk_base = p.chunk_base;
  const bool dec = p.flags & kDecoupled;
  const bool normalize = p.flags & kNormalize;
  const void* qn = dec ? a.q_rope : a.q;
  const void* kn = dec ? a.k_rope : a.k;
  void* dqn = dec ? a.dq_rope : a.dq;
  void* dkn = dec ? a.dk_rope : a.dk;
  void* dqd = dec ? a.dq : nullptr;
  void* dkd = dec ? a.dk : nullptr;
  const bool fast = mfma::supported(p, dtype);
  const int chunk = bwd_chunk(p, dtype);
  const int nchunks = (int)cdiv64(p.L, chunk);
  char* ws = (char*)a.workspace;
  float* partial = (float*)ws;
  ws += partial_bytes(p, dtype, chunk);
  float* St = (float*)ws;
  ws += state_bytes(p);
  float* dS = (float*)ws;
  ws += state_bytes(p);
  float* dSt = (float*)ws;
  ws += state_bytes(p);
  float* dkm = (float*)ws;
  ws += vec_bytes(p);
  float* tokscal = (float*)ws;
  const unsigned phases = phase_mask();
  const bool direct = fast && nchunks == 1;  // pass A stores the finished s*dS and dkm/L itself
  float* fm = direct ? dS : nullptr;
  float* fv = direct ? dkm : nullptr;
  if (phases & kPhaseBwdA) {
    if (mfma::bwd_a_supported(p, dtype)) {
      int rc = mfma::bwd_a(mfma::with_interleave(p, dtype, 4), dtype, qn, a.q, a.dout, a.s, a.km, dqn, dqd,
                           partial, chunk, nchunks, st, fm, fv);
      if (rc != kOk) return rc;
    } else if (fast) {
      // no fused kernel for this shape: token view and feature view as two kernels
      const int64_t rows = p.T * p.H;
      int rc = mfma::bwd_tokens(p, dtype, qn, a.q, a.dout, a.s, a.km, dqn, dqd, tokscal, rows, st);
      if (rc != kOk) return rc;
      if (normalize)
        mfma::scaled_state(p, dtype, qn, a.q, a.dout, tokscal, rows, partial, chunk, nchunks, st, fm, fv);
      else
        mfma::state(p, dtype, a.q, a.dout, a.q, partial, chunk, nchunks, st, fm, fv);
    } else {
      generic::transpose_state(p, a.s, St, st);
      generic::bwd_a(p, dtype, qn, a.q, a.dout, a.s, St, a.km, dqn, dqd, partial, chunk, nchunks, st);
    }
  }
  const bool fold = fast && !direct && !is_cross && dtype != kF32 && !mfma::pair_mode(p, dtype) &&
                    fold_reduce(p, nchunks, p.DV, p.DK);
  const int pchunk = mfma::bwd_a_supported(p, dtype) ? mfma::partial_chunk(p, dtype, 4, chunk) : chunk;
  if (!fold && !direct && (phases & kPhaseBwdReduce))
    generic::state_reduce(p, partial, pchunk, nchunks, dS, fast ? nullptr : dSt, dkm, st);
  if (phases & kPhaseBwdB) {
    if (fast) {
      // dk~_t = v_t (s dS)^T (+ dkm/L): contraction over dv, M(r=dv, c=dk) = dS[c][r]
      mfma::RowsJob jk{a.v, nullptr, dS, 1, p.DV, nullptr, (!dec && normalize) ? dkm : nullptr, dkn};
      if (p.flags & kElu1Grad) jk.gate = a.k;  // dk with respect to the keys before the feature map
      // dv_t = k~_t (s dS): contraction over dk
      mfma::RowsJob jv{kn, nullptr, dS, p.DV, 1, nullptr, nullptr, a.dv};
      jv.map_x = (p.flags & kElu1) != 0;  // (with kElu1: k itself is given before the map)
      if (fold) {  // both kernels sum the pass-A partials themselves (s dS, dkm/L)
        jk.mat = jv.mat = partial;
        jk.pchunk = jv.pchunk = pchunk;
        jk.pnchunks = jv.pnchunks = nchunks;
        jk.addvec = nullptr;
        jk.vec_is_add = !dec && normalize;
        jk.vec_out = dec ? dkm : nullptr;
      }
      // dkm arrives divided by the number of queries; the formula wants dkm / (number of keys)
      if (is_cross) jk.add_scale = (float)p.L / (float)pk.L;
      int rc;
      const Prob pki = mfma::with_interleave(pk, dtype, 2);
      if (p.DK == p.DV) {  // same shape: one launch
        rc = mfma::rows2(pki, dtype, jk, jv, p.DV, p.DK, st);
      } else {
        rc = mfma::rows(pki, dtype, jk, p.DV, p.DK, st);
        if (rc == kOk) rc = mfma::rows(pki, dtype, jv, p.DK, p.DV, st);
      }
      if (rc != kOk) return rc;
      // dk = dkm / (number of keys) in every key row; dkm arrives divided by the number of queries
      if (dec) generic::broadcast_rows(pk, dtype, dkm, dkd, st, is_cross ? (float)p.L / (float)pk.L : 1.f);
    } else {
      generic::bwd_b(pk, dtype, kn, a.v, dS, dSt, dkm, dkn, dkd, a.dv, st,
                     is_cross ? (float)p.L / (float)pk.L : 1.f);
    }
  }
  return kOk;
}

// ---- two queries sharing keys and values -------------------------------------------------------
// forward :  state partials of the whole DK x DV problem -> reduce (S, km) -> column halves S1, S2
//            -> one row launch with two jobs: o1 = (q1 S1) / (q1 . km + eps), o2 likewise
// backward:  pass A per query (dq_i, partials of dS_i and dkm_i) -> reduce -> dS = [dS1 | dS2],
//            dkm = dkm1 + dkm2 -> pass B of the whole problem (dk, dv): k and v are read once per
//            direction, dk is written once.
// Dense 16-bit problems whose whole and half shapes the matrix-core kernels cover, with the fused
// pass A for the half shape; the plain operator with the denominator.
static Prob half_values(const Prob& p) {
  Prob h = p;
  h.DV = p.DV / 2;
  return h;
}
bool pair_supported(const Prob& p, int dtype) {
  if (p.cu || dtype == kF32 || (p.DV & 1) || (p.flags & ~kNormalize) || !(p.flags & kNormalize)) return false;
  const Prob h = half_values(p);
  return mfma::supported(p, dtype) && mfma::supported(h, dtype) && mfma::bwd_a_supported(h, dtype) &&
         !mfma::pair_mode(h, dtype);
}
static size_t half_state_bytes(const Prob& p) { return state_bytes(half_values(p)); }
// partials | S1 | S2
size_t pair_fwd_workspace_bytes(const Prob& p, int dtype) {
  return partial_bytes(p, dtype, fwd_chunk(p, dtype)) + 2 * half_state_bytes(p);
}
// partials (half shape) | S1 | S2 | s dS1 | s dS2 | dkm1/L | dkm2/L | s dS | dkm/L
size_t pair_bwd_workspace_bytes(const Prob& p, int dtype) {
  const Prob h = half_values(p);
  return partial_bytes(h, dtype, bwd_chunk(h, dtype)) + 4 * half_state_bytes(p) + 3 * vec_bytes(p) + state_bytes(p);
}

int pair_forward(const Prob& p, int dtype, const PairFwdArgs& a, hipStream_t st) {
  if (!pair_supported(p, dtype)) {
    set_error("two queries on shared keys and values: dense fp16 / bf16 problems with the denominator whose "
              "whole (DK x DV) and half (DK x DV/2) shapes the matrix-core kernels cover");
    return kErrUnsupported;
  }
  const Prob h = half_values(p);
  const int chunk = fwd_chunk(p, dtype);
  const int nchunks = (int)cdiv64(p.L, chunk);
  char* ws = (char*)a.workspace;
  float* partial = (float*)ws;
  ws += partial_bytes(p, dtype, chunk);
  float* S1 = (float*)ws;
  ws += half_state_bytes(p);
  float* S2 = (float*)ws;
  const bool direct = nchunks == 1;
  mfma::state(mfma::with_interleave(p, dtype, 1), dtype, a.k, a.v, a.k, partial, chunk, nchunks, st,
              direct ? a.s : nullptr, direct ? a.km : nullptr);
  if (!direct)
    generic::state_reduce(p, partial, mfma::partial_chunk(p, dtype, 1, chunk), nchunks, a.s, nullptr, a.km, st);
  generic::split_columns(p, a.s, S1, S2, st);
  mfma::RowsJob j1{a.q[0], a.q[0], S1, h.DV, 1, a.km, nullptr, a.o[0]};
  mfma::RowsJob j2{a.q[1], a.q[1], S2, h.DV, 1, a.km, nullptr, a.o[1]};
  return mfma::rows2(mfma::with_interleave(h, dtype, 2), dtype, j1, j2, h.DK, h.DV, st);
}

int pair_backward(const Prob& p, int dtype, const PairBwdArgs& a, hipStream_t st) {
  if (!pair_supported(p, dtype)) {
    set_error("two queries on shared keys and values: dense fp16 / bf16 problems with the denominator whose "
              "whole (DK x DV) and half (DK x DV/2) shapes the matrix-core kernels cover");
    return kErrUnsupported;
  }
  const Prob h = half_values(p);
  const int chunk = bwd_chunk(h, dtype);
  const int nchunks = (int)cdiv64(h.L, chunk);
  char* ws = (char*)a.workspace;
  float* partial = (float*)ws;
  ws += partial_bytes(h, dtype, chunk);
  float* Sh[2];
  float* dSh[2];
  float* dkmh[2];
  for (int i = 0; i < 2; ++i, ws += half_state_bytes(p)) Sh[i] = (float*)ws;
  for (int i = 0; i < 2; ++i, ws += half_state_bytes(p)) dSh[i] = (float*)ws;
  for (int i = 0; i < 2; ++i, ws += vec_bytes(p)) dkmh[i] = (float*)ws;
  float* dkm = (float*)ws;
  ws += vec_bytes(p);
  float* dS = (float*)ws;
  generic::split_columns(p, a.s, Sh[0], Sh[1], st);
  const bool direct = nchunks == 1;
  const int pchunk = mfma::partial_chunk(h, dtype, 4, chunk);
  for (int i = 0; i < 2; ++i) {  // the partial buffer serves both queries in turn (one stream)
    int rc = mfma::bwd_a(mfma::with_interleave(h, dtype, 4), dtype, a.q[i], a.q[i], a.dout[i], Sh[i], a.km,
                         a.dq[i], nullptr, partial, chunk, nchunks, st, direct ? dSh[i] : nullptr,
                         direct ? dkmh[i] : nullptr);
    if (rc != kOk) return rc;
    if (!direct) generic::state_reduce(h, partial, pchunk, nchunks, dSh[i], nullptr, dkmh[i], st);
  }
  generic::join_columns(p, dSh[0], dSh[1], dkmh[0], dkmh[1], dS, dkm, st);
  // dk_t = v_t (s dS)^T + dkm/L, dv_t = k_t (s dS)
  mfma::RowsJob jk{a.v, nullptr, dS, 1, p.DV, nullptr, dkm, a.dk};
  mfma::RowsJob jv{a.k, nullptr, dS, p.DV, 1, nullptr, nullptr, a.dv};
  const Prob pi = mfma::with_interleave(p, dtype, 2);
  if (p.DK == p.DV) return mfma::rows2(pi, dtype, jk, jv, p.DV, p.DK, st);
  int rc = mfma::rows(pi, dtype, jk, p.DV, p.DK, st);
  if (rc == kOk) rc = mfma::rows(pi, dtype, jv, p.DK, p.DV, st);
  return rc;
}

}  // namespace plan
}  // namespace fbla
