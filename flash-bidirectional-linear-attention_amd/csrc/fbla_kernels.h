// Internal interface between the C-ABI layer (fbla_api.hip) and the kernel files.
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

namespace generic {
size_t fwd_workspace_bytes(const Prob& p);
size_t bwd_workspace_bytes(const Prob& p);
int forward(const Prob& p, int dtype, const FwdArgs& a, hipStream_t st);
int backward(const Prob& p, int dtype, const BwdArgs& a, hipStream_t st);
}  // namespace generic

}  // namespace fbla
