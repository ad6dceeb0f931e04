// Internal interface between the C-ABI layer (fbla_api.hip), the plan
// (fbla_plan.hip) and the kernel files.
#pragma once
#include "fbla_common.h"

namespace fbla {

struct FwdArgs {
  const void *q, *k, *v, *q_rope, *k_rope;
  void* o;
  float* s;   // [N*H, DK, DV] fp32 state, written
  float* km;  // [N*H, DK] fp32 key mean, written
  void* workspace;
  size_t workspace_bytes;
};

struct BwdArgs {
  const void *q, *k, *v, *q_rope, *k_rope, *dout;
  const float* s;
  const float* km;
  void *dq, *dk, *dv, *dq_rope, *dk_rope;
  void* workspace;
  size_t workspace_bytes;
};

// Kernel phases of one entry point, selectable for per-kernel timing
// (fbla_set_phase_mask).  Default: all.
enum Phase : unsigned {
  kPhaseFwdState = 1u,    // per-chunk partial K^T V and sum k
  kPhaseFwdReduce = 2u,   // fixed-order reduce of the partials
  kPhaseFwdOutput = 4u,   // o = (q S)/z
  kPhaseBwdA = 8u,        // dq + partial dS, dkm
  kPhaseBwdReduce = 16u,  // reduce of the backward partials
  kPhaseBwdB = 32u,       // dk, dv
  kPhaseAll = 63u,
};
unsigned phase_mask();

// Two queries that share keys and values (PolaFormer's same-sign / opposite-sign pairing): the first
// attends to the value columns [0, DV/2), the second to [DV/2, DV).  o, dout, dq are pairs of
// [.., DK] / [.., DV/2] tensors; k, v, dk, dv and the state are those of the whole DK x DV problem.
struct PairFwdArgs {
  const void *q[2], *k, *v;
  void* o[2];
  float* s;   // [N*H, DK, DV]
  float* km;  // [N*H, DK]
  void* workspace;
  size_t workspace_bytes;
};
struct PairBwdArgs {
  const void *q[2], *k, *v, *dout[2];
  const float* s;
  const float* km;
  void *dq[2], *dk, *dv;
  void* workspace;
  size_t workspace_bytes;
};

// The sequence of kernels behind each entry point.
namespace plan {
bool pair_supported(const Prob& p, int dtype);
size_t pair_fwd_workspace_bytes(const Prob& p, int dtype);
size_t pair_bwd_workspace_bytes(const Prob& p, int dtype);
int pair_forward(const Prob& p, int dtype, const PairFwdArgs& a, hipStream_t st);
int pair_backward(const Prob& p, int dtype, const PairBwdArgs& a, hipStream_t st);
size_t fwd_workspace_bytes(const Prob& p, int dtype);
size_t bwd_workspace_bytes(const Prob& p, int dtype);
int forward(const Prob& p, int dtype, const FwdArgs& a, hipStream_t st);
int backward(const Prob& p, int dtype, const BwdArgs& a, hipStream_t st);
}  // namespace plan

// Shape-generic FMA kernels (fbla_generic.hip).
namespace generic {
int state_chunk(const Prob& p);
void state_partial(const Prob& p, int dtype, const void* kn, const void* v, const void* kd,
                   float* partial, int chunk, int nchunks, hipStream_t st);
void state_reduce(const Prob& p, const float* partial, int chunk, int nchunks, float* mat,
                  float* mat_t, float* vec, hipStream_t st);
void transpose_state(const Prob& p, const float* mat, float* mat_t, hipStream_t st);
// `count` matrices of rs x cs elements (2 or 4 bytes each) into matrices of rd x cd: the common part is copied,
// the rest of the destination is zero
void resize_matrices(const void* src, int64_t rs, int cs, void* dst, int64_t rd, int cd, int64_t count, int elem_bytes,
                     hipStream_t st);
// p.DV even: the column halves of a [N*H, DK, DV] matrix as two [N*H, DK, DV/2] matrices, and back
// (join also adds two [N*H, DK] vectors when `vec` is given)
void split_columns(const Prob& p, const float* mat, float* lo, float* hi, hipStream_t st);
void join_columns(const Prob& p, const float* lo, const float* hi, const float* vec_lo, const float* vec_hi,
                  float* mat, float* vec, hipStream_t st);
void output(const Prob& p, int dtype, const void* qn, const void* qd, const float* S,
            const float* km, void* o, hipStream_t st);
void bwd_a(const Prob& p, int dtype, const void* qn, const void* qd, const void* dout,
           const float* S, const float* St, const float* km, void* dqn, void* dqd, float* partial,
           int chunk, int nchunks, hipStream_t st);
// dkm_scale: the vector arrives divided by the number of queries; with another number of keys
// the formula wants it divided by that (factor Lq / Lk)
void bwd_b(const Prob& p, int dtype, const void* kn, const void* v, const float* dS,
           const float* dSt, const float* dkm, void* dkn, void* dkd, void* dv, hipStream_t st,
           float dkm_scale = 1.f);
void broadcast_rows(const Prob& p, int dtype, const float* vec, void* out, hipStream_t st, float factor = 1.f);
// perm[r] = index of the sequence with the r-th largest length (ties by index)
void rank_sequences(const Prob& p, int32_t* perm, hipStream_t st);
// base[0..N]: exclusive prefix sums of the sequences' numbers of chunks of `chunk` tokens
void chunk_bases(const Prob& p, int chunk, int32_t* base, hipStream_t st);
}  // namespace generic

// MFMA kernels for 16-bit inputs (fbla_mfma.hip).
namespace mfma {
struct RowsJob {
  const void* x;        // [rows][DR] contracted operand
  const void* xden;     // [rows][DR] rows dotted with km for z (== x unless decoupled); null: z = 1
  const float* mat;     // per (sequence, head): element (r, c) at mat[r*ld_r + c*ld_c]
  int ld_r, ld_c;
  const float* km;      // per (sequence, head) [DR]; used when xden != null
  const float* addvec;  // per (sequence, head) [DC] added to every row, or null
  void* out;            // [rows][DC]
  // pnchunks > 0: `mat` is instead the partial buffer written by the state kernel /
  // backward pass A with chunking (pchunk, pnchunks); the kernel sums the partials
  // itself (matrix times the state scale, vector times 1/len).  The vector is km
  // (when xden is set) or the row added to the output (vec_is_add).  mat_out /
  // vec_out (nullable) receive the reduced matrix [DK*DV] and vector [DK].
  int pchunk = 0, pnchunks = 0;
  bool vec_is_add = false;
  float* mat_out = nullptr;
  float* vec_out = nullptr;
  float add_scale = 1.f;  // factor on addvec (queries / keys when their numbers differ)
  bool map_x = false;          // kElu1 together with kElu1Grad: this job's x rows arrive before the map
  const void* gate = nullptr;  // [rows][DC] mapped rows phi(x): the output is multiplied by min(gate, 1), the
                               // derivative of phi (kElu1Grad; the dk job of the backward; rows before the map
                               // when kElu1 is set as well), or null
};
bool supported(const Prob& p, int dtype);
bool bwd_a_supported(const Prob& p, int dtype);
// dense 32 x 32 heads: the row-parallel kernels take two tokens per row and need the finished
// matrices (no partial sums in their prologue)
bool pair_mode(const Prob& p, int dtype);
// block_stats: the launch that also writes piecewise attention's block statistics
int state_chunk(const Prob& p, bool block_stats = false);
int bwd_a_chunk(const Prob& p);
int rows_chunk(const Prob& p, int DR, int DC);
// Tokens per partial as a reduction must count them (`kernel_bit`: 1 the state kernel, 4 backward
// pass A): the kernel's chunk, or the step of the interleaved walk when the workgroups of a head
// take interleaved steps.
int partial_chunk(const Prob& p, int dtype, int kernel_bit, int chunk);
// The problem with the interleaved walk switched on for the kernel `kernel_bit` (1 the state
// kernel, 2 the row-parallel kernels, 4 backward pass A) where it applies: dense 16-bit heads
// tiled 64 x 64.  Only for callers that treat the partials as an unordered set to be summed
// (partial_chunk tells how many of them a sequence of a given length has).
Prob with_interleave(const Prob& p, int dtype, int kernel_bit);
// fin_mat / fin_vec (only with nchunks == 1): store the finished, scaled matrix [N*H,DK,DV] and
// vector [N*H,DK] directly instead of a partial (no reduce step needed)
void state(const Prob& p, int dtype, const void* kn, const void* v, const void* kd, float* partial,
           int chunk, int nchunks, hipStream_t st, float* fin_mat = nullptr, float* fin_vec = nullptr);
// The state partials (as `state` with kd = kn, no final store) plus the block statistics of
// piecewise attention: per 64-token block the mean key kc [N*H, NT, DK] and the value sum
// vc [N*H, NT, DV] (fp32).  chunk must be a multiple of 64.
void state_with_block_stats(const Prob& p, int dtype, const void* k, const void* v, float* partial,
                            int chunk, int nchunks, float* kc, float* vc, int NT, hipStream_t st);
// out_t = (x_t M) / (xden_t . km + eps) + addvec   with M of shape DR x DC
int rows(const Prob& p, int dtype, const RowsJob& job, int DR, int DC, hipStream_t st);
int rows2(const Prob& p, int dtype, const RowsJob& job0, const RowsJob& job1, int DR, int DC,
          hipStream_t st);
// two-kernel form of backward pass A (the 16-bit decoupled operator with a 128-wide side, packed
// batches of more than 65536 heads with one, fp32 inputs): qn / dqn are the rows of the numerator and their gradient
// (q_rope, dq_rope when decoupled; then qd = q, dqd = dq), otherwise qn == qd and dqd is unused.
// bwd_tokens writes dq and tokscal = [1/z_t | dz_t] per (token, head) row, scaled_state
// accumulates the partials of dS = sum_t q_t^T (dO_t / z_t) and dkm = sum_t dz_t q_t
int bwd_tokens(const Prob& p, int dtype, const void* qn, const void* qd, const void* dout, const float* S,
               const float* km, void* dqn, void* dqd, float* tokscal, int64_t total_rows, hipStream_t st);
void scaled_state(const Prob& p, int dtype, const void* qn, const void* qd, const void* dout,
                  const float* tokscal, int64_t total_rows, float* partial, int chunk, int nchunks,
                  hipStream_t st, float* fin_mat = nullptr, float* fin_vec = nullptr);
// backward pass A: dq~ (and dq when decoupled) + per-chunk partials of dS and dkm
int bwd_a(const Prob& p, int dtype, const void* qn, const void* qd, const void* dout, const float* S,
          const float* km, void* dqn, void* dqd, float* partial, int chunk, int nchunks,
          hipStream_t st, float* fin_mat = nullptr, float* fin_vec = nullptr);
}  // namespace mfma

namespace mfma32 {
// fp32 inputs on v_mfma_f32_32x32x2_f32: head dims that are multiples of 4 up to 64 (plain and
// decoupled) or up to 128 (plain).  Called through the mfma:: entry points, which dispatch on the dtype.
bool supported(const Prob& p);
void state(const Prob& p, const float* kn, const float* v, const float* kd, float* partial,
           const float* tokscal, int64_t total_rows, int chunk, int nchunks, hipStream_t st, float* fin_mat,
           float* fin_vec);
int rows(const Prob& p, const mfma::RowsJob& job, const mfma::RowsJob* job2, int dr, int dc, hipStream_t st);
int bwd_tokens(const Prob& p, const float* qn, const float* qd, const float* dout, const float* S,
               const float* km, float* dqn, float* dqd, float* tokscal, int64_t total_rows, hipStream_t st);
// Heads with a side above 64 (fbla_mfma32w.hip): tiled 128 x 128, head dims that are multiples of 4 up
// to 128, the plain operator (not decoupled).  The functions above hand such problems over.
bool wide(const Prob& p);
bool wide_supported(const Prob& p);
void wide_state(const Prob& p, const float* kn, const float* v, float* partial, const float* tokscal,
                int64_t total_rows, int chunk, int nchunks, hipStream_t st, float* fin_mat, float* fin_vec);
int wide_rows(const Prob& p, const mfma::RowsJob& job, const mfma::RowsJob* job2, int dr, int dc, hipStream_t st);
int wide_bwd_tokens(const Prob& p, const float* q, const float* dout, const float* S, const float* km, float* dq,
                    float* tokscal, int64_t total_rows, hipStream_t st);
}  // namespace mfma32

// The callers' feature map elu(x) + 1 and its derivative (fbla_feature.hip).
namespace feature {
// y0 = elu(x0) + 1 over n0 elements and y1 = elu(x1) + 1 over n1 elements, one launch
void elu1_fwd(const void* x0, void* y0, int64_t n0, const void* x1, void* y1, int64_t n1, int dtype,
              hipStream_t st);
// dx = g * (x > 0 ? 1 : exp(x))
void elu1_bwd(const void* x, const void* g, void* dx, int64_t n, int dtype, hipStream_t st);
}  // namespace feature

// Piecewise (PISA) attention, forward only (fbla_piecewise.hip).
namespace piecewise {
size_t chunk_reduce_workspace_bytes(int64_t BH, int64_t T, int K, int V, int chunk, int dtype,
                                    bool per_chunk);
int chunk_reduce(const void* q, const void* k, const void* v, float* qc, float* kc, float* vc,
                 float* h, float* h_norm, void* workspace, int64_t BH, int64_t T, int K, int V,
                 int chunk, float pnorm, int dtype, hipStream_t st);
// top-NS key blocks per query block from the block means (ascending block order)
bool select_blocks_supported(int NT, int K);
int select_blocks(const float* qc, const float* kc, const float* bias, int32_t* indices, int64_t BH,
                  int NT, int K, int NS, float scale, hipStream_t st);
bool attention_supported(int K, int V, int block, int dtype);
size_t attention_workspace_bytes(int64_t BH, int64_t T, int K, int V, int block);
int attention(const void* q, const void* k, const void* v, const float* kc, const float* vc,
              const float* h, const int32_t* indices, void* o, void* workspace, int64_t BH, int64_t T,
              int K, int V, int block, int NS, float scale, int dtype, hipStream_t st);
// the same operator for every head dim up to 128, every block size and fp32 inputs (fp32 FMAs,
// no workspace): what `attention` does not cover
bool attention_generic_supported(int64_t T, int K, int V, int block, int dtype);
int attention_generic(const void* q, const void* k, const void* v, const float* kc, const float* vc,
                      const float* h, const int32_t* indices, void* o, int64_t BH, int64_t T, int K, int V,
                      int block, int NS, float scale, int dtype, hipStream_t st);
}  // namespace piecewise

}  // namespace fbla
