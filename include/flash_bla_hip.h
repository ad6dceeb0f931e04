/*
 * flash_bla_hip.h -- C ABI of libfbla_hip.so: bidirectional (non-causal) linear
 * attention for AMD gfx950 (MI355X).
 *
 * The reference (fla-org/flash-bidirectional-linear-attention, `flash_bla`) has
 * no native layer: its operators are torch.autograd.Function classes that launch
 * Triton kernels.  Each entry point below replaces the kernel launches made by
 * one of those Functions; the Python operator layer keeps the reference's
 * signatures and binds these symbols with ctypes.
 *
 * Conventions
 *   - every pointer is a DEVICE pointer unless stated otherwise; the library
 *     never allocates, frees or retains device memory: outputs and the workspace
 *     are provided by the caller (size from the *_workspace_bytes queries);
 *   - work is enqueued on `stream` (a hipStream_t passed as void*); no call
 *     synchronises the device;
 *   - return value 0 = success, negative = error (fbla_last_error() gives the
 *     text for the calling thread); no C++ exception crosses the boundary;
 *   - dense tensors are contiguous [B,H,L,D]; packed tensors are contiguous
 *     [T_total,H,D] with int32 cu_seqlens[N+1] on the device;
 *   - the state tensors s [B*H,DK,DV] (or [N*H,DK,DV]) and km [..,DK] are fp32.
 *     s already includes `scale`; km is the mean key.  Forward writes them,
 *     backward reads them (the reference saves the same two tensors in its
 *     autograd context: linear_attn/fused.py:395);
 *   - reductions over tokens are two-stage and fixed-order: results are
 *     bit-identical from run to run.
 */
#ifndef FLASH_BLA_HIP_H
#define FLASH_BLA_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* element type of q/k/v/o and of the gradients */
#define FBLA_F16 0
#define FBLA_BF16 1
#define FBLA_F32 2

/* flags */
#define FBLA_NORMALIZE 1     /* o = (q S)/(q.km + eps); clear = simple_la (no denominator) */
#define FBLA_DECOUPLED 2     /* numerator from q_rope/k_rope, denominator from q/k */
#define FBLA_DEFAULT_SCALE 4 /* packed layout only: scale = 1/len_i per sequence */
#define FBLA_ELU1_QK 8       /* q and k are given BEFORE the callers' feature map
                              * phi(x) = elu(x) + 1 (layers/linfusion.py:88-89, layers/mlla.py:74-75) and the
                              * kernels apply it as they load them; fp16 / bf16, DK = DV = 64, not decoupled
                              * (FBLA_ERR_UNSUPPORTED otherwise); the backward entry points take it together
                              * with FBLA_ELU1_GRAD only */
#define FBLA_ELU1_GRAD 16    /* backward entry points only: q and k are the MAPPED tensors phi(x) = elu(x) + 1 (what
                              * the forward consumed and saved) and dq, dk are wanted with respect to x: the
                              * kernels multiply them by phi'(x) = min(phi(x), 1) as they write them, which
                              * replaces the autograd of `F.elu(x) + 1.0` (two elementwise launches per call).
                              * Together with FBLA_ELU1_QK, q and k are given before the map here as well and the
                              * backward kernels map them on load (no mapped copies exist anywhere).
                              * fp16 / bf16, DK = DV = 64, not decoupled (FBLA_ERR_UNSUPPORTED otherwise) */

/* error codes */
#define FBLA_OK 0
#define FBLA_ERR_BAD_ARG (-1)
#define FBLA_ERR_UNSUPPORTED (-2)
#define FBLA_ERR_WORKSPACE (-3)
#define FBLA_ERR_LAUNCH (-4)

/* Library version (major*10000 + minor*100 + patch). */
int fbla_version(void);

/* Profiling aid with no counterpart in the reference: restrict the entry points
 * called from this thread to a subset of their kernels so that one kernel can be
 * timed in isolation (bit 0 forward partial state, 1 forward state reduce,
 * 2 forward output, 3 backward pass A, 4 backward reduce, 5 backward pass B).
 * 0 restores the default (all kernels).  Skipped kernels leave their outputs
 * untouched, so results are only meaningful with the default mask.  Ignored unless
 * the process was started with FBLA_ALLOW_PHASE_MASK=1 in its environment. */
void fbla_set_phase_mask(unsigned mask);

/* Message of the last error raised on the calling thread ("" if none). */
const char* fbla_last_error(void);

/* Workspace (bytes) needed by fbla_la_fwd (pass=0) / fbla_la_bwd (pass=1) for a
 * dense problem.  Replaces the torch.empty temporaries of
 * linear_attn/fused.py:362-363,422-423 (which grow with L/32; ours do not). */
size_t fbla_la_workspace_bytes(int pass, int64_t B, int64_t H, int64_t L, int DK, int DV,
                               int dtype, int flags);

/* Dense forward.  Replaces the launches in
 *   LinearAttnFunction.forward        flash_bla/ops/linear_attn/fused.py:352-398
 *   SimpleLinearAttnFunction.forward  flash_bla/ops/simple_la/fused.py:495-535   (flags without FBLA_NORMALIZE)
 *   DecoupledLAFunction.forward       flash_bla/ops/linear_attn/decoupled.py:413-460 (FBLA_DECOUPLED)
 * q,k,(q_rope,k_rope): [B,H,L,DK]; v,o: [B,H,L,DV]; q_rope/k_rope NULL unless decoupled. */
int fbla_la_fwd(const void* q, const void* k, const void* v, const void* q_rope,
                const void* k_rope, void* o, float* s, float* km, void* workspace,
                size_t workspace_bytes, int64_t B, int64_t H, int64_t L, int DK, int DV, int dtype,
                int flags, float scale, float eps, void* stream);

/* Dense backward.  Replaces the launches in
 *   LinearAttnFunction.backward        flash_bla/ops/linear_attn/fused.py:400-453
 *   SimpleLinearAttnFunction.backward  flash_bla/ops/simple_la/fused.py:537-626
 *   DecoupledLAFunction.backward       flash_bla/ops/linear_attn/decoupled.py:462-509
 * `o` is not an input: o.dO is recomputed from q and s.  dq_rope/dk_rope are
 * written only when decoupled (then dq/dk receive the denominator gradients). */
int fbla_la_bwd(const void* q, const void* k, const void* v, const void* q_rope,
                const void* k_rope, const void* dout, const float* s, const float* km, void* dq,
                void* dk, void* dv, void* dq_rope, void* dk_rope, void* workspace,
                size_t workspace_bytes, int64_t B, int64_t H, int64_t L, int DK, int DV, int dtype,
                int flags, float scale, float eps, void* stream);

/* Dense forward that allocates nothing.  No counterpart in the reference: it is for callers
 * that cannot allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc) and have no workspace to hand over.  Same arguments,
 * arithmetic and results as fbla_la_fwd, but the workspace is a fixed array of
 * FBLA_STATIC_SCRATCH_BYTES inside the library's device image (each GPU the library runs on
 * holds one copy until the process ends).  A problem whose fbla_la_workspace_bytes(0, ...)
 * exceeds that returns FBLA_ERR_WORKSPACE.  The call makes no hipMalloc / hipFree and no
 * allocating library call.  All calls on one GPU share the array: calls that overlap on one
 * GPU (two streams, two threads) race; serialise them or use fbla_la_fwd.  The first call on a
 * device looks up the array's address (hipGetSymbolAddress, which may load the code object) and
 * sets the kernels' LDS attributes: make one eager call per device and problem shape before
 * recording calls into a HIP graph. */
#define FBLA_STATIC_SCRATCH_BYTES (16u << 20)
size_t fbla_static_scratch_bytes(void);
int fbla_la_fwd_static(const void* q, const void* k, const void* v, const void* q_rope,
                       const void* k_rope, void* o, float* s, float* km, int64_t B, int64_t H,
                       int64_t L, int DK, int DV, int dtype, int flags, float scale, float eps,
                       void* stream);

/* Two queries on shared keys and values, dense, with the denominator.  Replaces the two operator
 * calls of PolaLinearAttention.forward (flash_bla/layers/polaformer.py:89-90:
 *   x_sim = linear_attention(q_sim, k, v1),  x_opp = linear_attention(q_opp, k, v2)
 * with v1 | v2 the two halves of the value channels), which read k twice forward and twice
 * backward and leave the sum of the two dk to autograd.  Here
 *   S = scale * K^T [v1 | v2]  (one pass over k and v),  km = mean k,
 *   o1 = (q1 S[:, :DV/2]) / (q1 . km + eps),  o2 = (q2 S[:, DV/2:]) / (q2 . km + eps),
 * and the backward reads k and v once and writes dk = dk1 + dk2 once.
 * q1, q2, dq1, dq2, k, dk: [B,H,L,DK]; v, dv: [B,H,L,DV]; o1, o2, dout1, dout2: [B,H,L,DV/2];
 * s: [B,H,DK,DV], km: [B,H,DK] fp32.  fp16 / bf16, DK and DV/2 multiples of 8 up to 128 (the
 * workspace query returns 0 for anything else, the calls FBLA_ERR_UNSUPPORTED). */
size_t fbla_la_pair_workspace_bytes(int pass, int64_t B, int64_t H, int64_t L, int DK, int DV, int dtype);
int fbla_la_pair_fwd(const void* q1, const void* q2, const void* k, const void* v, void* o1, void* o2,
                     float* s, float* km, void* workspace, size_t workspace_bytes, int64_t B, int64_t H,
                     int64_t L, int DK, int DV, int dtype, float scale, float eps, void* stream);
int fbla_la_pair_bwd(const void* q1, const void* q2, const void* k, const void* v, const void* dout1,
                     const void* dout2, const float* s, const float* km, void* dq1, void* dq2, void* dk,
                     void* dv, void* workspace, size_t workspace_bytes, int64_t B, int64_t H, int64_t L,
                     int DK, int DV, int dtype, float scale, float eps, void* stream);

/* Dense problems with Lk key / value tokens and Lq query tokens per (batch, head), Lk != Lq:
 * q, dq: [B,H,Lq,DK]; k, dk: [B,H,Lk,DK]; v, dv: [B,H,Lk,DV]; o, dout: [B,H,Lq,DV]; km is the mean
 * over the Lk keys.  The reference has no counterpart: its dense kernels take one length from q
 * (linear_attn/fused.py:355) and read k, v out of bounds when the PVT-style blocks
 * (layers/focused_la.py:55,73-75, layers/polaformer.py) shorten the keys with sr_ratio > 1.
 * Flags as for fbla_la_fwd without FBLA_DECOUPLED (the decoupled operator has the pair of entry
 * points below); every dtype and head dim of fbla_la_fwd.  fbla_la_cross_workspace_bytes takes
 * FBLA_DECOUPLED in `flags` for the decoupled pair. */
size_t fbla_la_cross_workspace_bytes(int pass, int64_t B, int64_t H, int64_t Lq, int64_t Lk, int DK,
                                     int DV, int dtype, int flags);
int fbla_la_cross_fwd(const void* q, const void* k, const void* v, void* o, float* s, float* km,
                      void* workspace, size_t workspace_bytes, int64_t B, int64_t H, int64_t Lq,
                      int64_t Lk, int DK, int DV, int dtype, int flags, float scale, float eps,
                      void* stream);
int fbla_la_cross_bwd(const void* q, const void* k, const void* v, const void* dout, const float* s,
                      const float* km, void* dq, void* dk, void* dv, void* workspace,
                      size_t workspace_bytes, int64_t B, int64_t H, int64_t Lq, int64_t Lk, int DK,
                      int DV, int dtype, int flags, float scale, float eps, void* stream);

/* The decoupled operator with Lk != Lq: q, q_rope, dq, dq_rope: [B,H,Lq,DK]; k, k_rope, dk, dk_rope:
 * [B,H,Lk,DK]; v, dv: [B,H,Lk,DV]; o, dout: [B,H,Lq,DV].  No counterpart in the reference
 * (linear_attn/decoupled.py:413-509 takes one length from q).  Workspace: fbla_la_cross_workspace_bytes
 * with flags = FBLA_NORMALIZE | FBLA_DECOUPLED. */
int fbla_decoupled_cross_fwd(const void* q, const void* k, const void* q_rope, const void* k_rope,
                             const void* v, void* o, float* s, float* km, void* workspace,
                             size_t workspace_bytes, int64_t B, int64_t H, int64_t Lq, int64_t Lk, int DK,
                             int DV, int dtype, float scale, float eps, void* stream);
int fbla_decoupled_cross_bwd(const void* q, const void* k, const void* q_rope, const void* k_rope,
                             const void* v, const void* dout, const float* s, const float* km, void* dq,
                             void* dk, void* dq_rope, void* dk_rope, void* dv, void* workspace,
                             size_t workspace_bytes, int64_t B, int64_t H, int64_t Lq, int64_t Lk, int DK,
                             int DV, int dtype, float scale, float eps, void* stream);

/* Workspace for the packed (variable-length) entry points. */
size_t fbla_varlen_workspace_bytes(int pass, int64_t total_tokens, int64_t N, int64_t H,
                                   int64_t max_seqlen, int DK, int DV, int dtype, int flags);

/* Packed forward.  Replaces VarlenLinearAttnFunction.forward
 * (flash_bla/ops/linear_attn/varlen.py:339-422).  max_seqlen is an upper bound on
 * the sequence lengths and only sizes the launch; any value >= the true maximum
 * gives the same result (tests/ops/test_varlen_linear_attn.py:45-55).  With
 * FBLA_DEFAULT_SCALE each sequence uses 1/len_i (varlen.py:66) and `scale` is ignored.
 * s: [N*H,DK,DV], km: [N*H,DK] fp32. */
int fbla_varlen_fwd(const void* q, const void* k, const void* v, const int32_t* cu_seqlens,
                    void* o, float* s, float* km, void* workspace, size_t workspace_bytes,
                    int64_t total_tokens, int64_t N, int64_t H, int64_t max_seqlen, int DK, int DV,
                    int dtype, int flags, float scale, float eps, void* stream);

/* Packed backward.  Replaces VarlenLinearAttnFunction.backward (varlen.py:426-505). */
int fbla_varlen_bwd(const void* q, const void* k, const void* v, const int32_t* cu_seqlens,
                    const void* dout, const float* s, const float* km, void* dq, void* dk, void* dv,
                    void* workspace, size_t workspace_bytes, int64_t total_tokens, int64_t N,
                    int64_t H, int64_t max_seqlen, int DK, int DV, int dtype, int flags,
                    float scale, float eps, void* stream);

/* ---- piecewise (PISA) attention, forward only --------------------------------
 * Tensors are contiguous [BH, T, K] / [BH, T, V] (batch and heads flattened). */

/* Workspace of fbla_chunk_reduce (with_norm != 0 when h_norm is requested). */
size_t fbla_chunk_reduce_workspace_bytes(int64_t BH, int64_t T, int K, int V, int chunk, int dtype,
                                         int with_norm);

/* Block statistics of the linear branch.  Replaces fused_chunk_reduce /
 * fused_chunk_reduce_kernel (flash_bla/ops/piecewise_attn/kernel.py:89-128,152-176).
 * With NT = ceil(T/chunk): qc, kc [BH,NT,K] = chunk means of q, k; vc [BH,NT,V] = chunk
 * sums of v; h [BH,K,V] = sum_c (K_c - kc_c)^T V_c; h_norm [BH,NT] (optional, may be
 * NULL) = p-norm of each chunk's (K_c - kc_c)^T V_c (kernel.py:172-174).  All outputs
 * are fp32 (the reference stores them in the input dtype). */
int fbla_chunk_reduce(const void* q, const void* k, const void* v, float* qc, float* kc, float* vc,
                      float* h, float* h_norm, void* workspace, size_t workspace_bytes, int64_t BH,
                      int64_t T, int K, int V, int chunk, float p_norm, int dtype, void* stream);

/* Block selection.  Replaces the score matrix and torch.topk of the wrapper
 * (flash_bla/ops/piecewise_attn/kernel.py:304-318): for every query block the NS key blocks
 * with the largest qc . kc * scale (+ log(bias + 1e-5) when bias [BH,NT], the h_norm output
 * of fbla_chunk_reduce, is given; kernel.py:314-315 applies a softmax on top, which does not
 * change the order).  qc, kc: fp32 [BH,NT,K] from fbla_chunk_reduce; indices: int32
 * [BH,NT,NS], written in ascending block order (torch.topk orders by score; the attention
 * result does not depend on the order); ties at the threshold go to the lower block index.
 * K in [1,128]; the scores of 16 query blocks against all NT key blocks must fit LDS
 * (NT up to about 2000). */
int fbla_select_blocks(const float* qc, const float* kc, const float* bias, int32_t* indices,
                       int64_t BH, int64_t NT, int K, int NS, float scale, void* stream);

/* Workspace of fbla_piecewise_fwd; 0 when the shape is not supported (a head dim above 128, or so
 * many blocks that their selection flags do not fit LDS). */
size_t fbla_piecewise_workspace_bytes(int64_t BH, int64_t T, int K, int V, int block, int dtype);

/* Piecewise attention forward.  Replaces piecewise_sparse_attention_fwd_kernel
 * (kernel.py:189-292): exact softmax attention over the NS selected key blocks of every
 * query block of `block` tokens (indices: int32 [BH, NT, NS], NT = ceil(T / block)), the
 * remaining blocks through their mean key / value sum (zeroth order) and h (first order).
 * kc, vc, h are the fp32 outputs of fbla_chunk_reduce with chunk = block.  fp16 / bf16 with
 * block = 16, 32 or a multiple of 64 run on the MFMA kernel (K, V other than 64 / 128 through
 * zero-widened copies in the workspace); other block sizes and fp32 inputs run on a shape-generic
 * fp32 kernel (same results to rounding, one to two orders of magnitude slower, no workspace
 * used).  The reference takes the same domain through BK = min(128, next_pow2(K))
 * (kernel.py:296-308). */
int fbla_piecewise_fwd(const void* q, const void* k, const void* v, const float* kc, const float* vc,
                       const float* h, const int32_t* indices, void* o, void* workspace,
                       size_t workspace_bytes, int64_t BH, int64_t T, int K, int V, int block, int NS,
                       float scale, int dtype, void* stream);

/* The feature map of the reference's blocks, phi(x) = elu(x) + 1, for the queries and the
 * keys in one launch.  Replaces the two elementwise torch kernels per tensor of
 * flash_bla/layers/linfusion.py:88-89, mlla.py:74-75 and rala.py:52-53 (`F.elu(x) + 1.0`), with
 * torch's rounding (elu in fp32 rounded to the element type, then + 1 rounded again).
 * x0/y0 hold n0 elements, x1/y1 n1 (either count may be 0); y may alias x.  Any dtype of the
 * FBLA_* element types; pointers 16-byte aligned. */
int fbla_elu1_fwd(const void* x0, void* y0, int64_t n0, const void* x1, void* y1, int64_t n1, int dtype,
                  void* stream);

/* Its derivative: dx = dy * (x > 0 ? 1 : exp(x)), what autograd computes for `F.elu(x) + 1.0`. */
int fbla_elu1_bwd(const void* x, const void* dy, void* dx, int64_t n, int dtype, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* FLASH_BLA_HIP_H */
