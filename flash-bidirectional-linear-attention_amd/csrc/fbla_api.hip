// C-ABI layer of libfbla_hip.so: argument checks, kernel-family dispatch and
// error reporting.  Declarations and the reference call sites each entry point
// replaces are in include/flash_bla_hip.h.
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>

#include <atomic>
#include <initializer_list>
#include <mutex>

#include "../../include/flash_bla_hip.h"
#include "fbla_kernels.h"

namespace fbla {

static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

static thread_local unsigned g_phase_mask = kPhaseAll;
unsigned phase_mask() { return g_phase_mask; }

static int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    set_error("%s: kernel launch failed: %s", what, hipGetErrorString(e));
    return kErrLaunch;
  }
  return kOk;
}

static int check_dims(const char* what, int64_t N, int64_t H, int64_t L, int DK, int DV,
                      int dtype, int flags) {
  if (N < 0 || H <= 0 || L < 0) {
    set_error("%s: bad sizes N=%lld H=%lld L=%lld", what, (long long)N, (long long)H, (long long)L);
    return kErrBadArg;
  }
  if (DK < 1 || DK > 128 || DV < 1 || DV > 128) {
    set_error("%s: head dims must be in [1,128], got DK=%d DV=%d", what, DK, DV);
    return kErrUnsupported;
  }
  if (dtype != kF16 && dtype != kBF16 && dtype != kF32) {
    set_error("%s: unknown dtype %d", what, dtype);
    return kErrBadArg;
  }
  if (flags & ~kPublicFlags) {
    set_error("%s: unknown flag bits 0x%x", what, flags & ~kPublicFlags);
    return kErrBadArg;
  }
  if ((flags & kDecoupled) && !(flags & kNormalize)) {
    set_error("%s: FBLA_DECOUPLED requires FBLA_NORMALIZE", what);
    return kErrBadArg;
  }
  if (N * H > 0x7fffffffLL / 4 || L > 0x7fffffffLL / 2) {
    set_error("%s: problem too large for 32-bit grid indexing", what);
    return kErrUnsupported;
  }
  return kOk;
}

// The kernels move 16-byte pieces of rows.
static int check_aligned(const char* what, std::initializer_list<const void*> ptrs) {
  for (const void* ptr : ptrs)
    if (reinterpret_cast<uintptr_t>(ptr) & 15) {
      set_error("%s: tensor pointers must be 16-byte aligned", what);
      return kErrBadArg;
    }
  return kOk;
}

static Prob make_prob(const int32_t* cu, int64_t N, int64_t H, int64_t L, int64_t T, int DK, int DV,
                      int flags, float scale, float eps) {
  Prob p;
  p.cu = cu;
  p.perm = nullptr;
  p.chunk_base = nullptr;
  p.N = (int)N;
  p.H = (int)H;
  p.L = (int)L;
  p.Lk = 0;
  p.T = T;
  p.DK = DK;
  p.DV = DV;
  p.scale = scale;
  p.eps = eps;
  p.flags = flags;
  return p;
}

static size_t workspace_bytes(const Prob& p, int dtype, int pass) {
  return pass == 0 ? plan::fwd_workspace_bytes(p, dtype) : plan::bwd_workspace_bytes(p, dtype);
}

static int run_fwd(const char* what, const Prob& p, int dtype, const FwdArgs& a, hipStream_t st) {
  if ((int64_t)p.N * p.H == 0 || p.L == 0) return kOk;
  if (check_aligned(what, {a.q, a.k, a.v, a.q_rope, a.k_rope, a.o, a.s, a.km, a.workspace}) != kOk)
    return kErrBadArg;
  const size_t need = workspace_bytes(p, dtype, 0);
  if (a.workspace_bytes < need || (need && !a.workspace)) {
    set_error("%s: workspace too small (%zu < %zu bytes)", what, a.workspace_bytes, need);
    return kErrWorkspace;
  }
  int rc = plan::forward(p, dtype, a, st);
  if (rc != kOk) return rc;
  return check_launch(what);
}

static int run_bwd(const char* what, const Prob& p, int dtype, const BwdArgs& a, hipStream_t st) {
  if ((int64_t)p.N * p.H == 0 || p.L == 0) return kOk;
  if (check_aligned(what, {a.q, a.k, a.v, a.q_rope, a.k_rope, a.dout, a.s, a.km, a.dq, a.dk, a.dv, a.dq_rope,
                           a.dk_rope, a.workspace}) != kOk)
    return kErrBadArg;
  const size_t need = workspace_bytes(p, dtype, 1);
  if (a.workspace_bytes < need || (need && !a.workspace)) {
    set_error("%s: workspace too small (%zu < %zu bytes)", what, a.workspace_bytes, need);
    return kErrWorkspace;
  }
  int rc = plan::backward(p, dtype, a, st);
  if (rc != kOk) return rc;
  return check_launch(what);
}

}  // namespace fbla

using namespace fbla;

extern "C" {

int fbla_version(void) { return 100; }

// Only honoured when the process opted in through the environment: a caller cannot switch kernels
// off by accident, and a mask left set by a profiling script that died cannot outlive its process.
void fbla_set_phase_mask(unsigned mask) {
  static const bool allowed = [] { const char* v = getenv("FBLA_ALLOW_PHASE_MASK"); return v && v[0] == '1'; }();
  g_phase_mask = (allowed && mask) ? mask : kPhaseAll;
}

const char* fbla_last_error(void) { return g_err; }

size_t fbla_la_workspace_bytes(int pass, int64_t B, int64_t H, int64_t L, int DK, int DV, int dtype,
                               int flags) {
  if (check_dims("fbla_la_workspace_bytes", B, H, L, DK, DV, dtype, flags) != kOk) return 0;
  Prob p = make_prob(nullptr, B, H, L, B * L, DK, DV, flags, 1.f, 0.f);
  return workspace_bytes(p, dtype, pass);
}

int fbla_la_fwd(const void* q, const void* k, const void* v, const void* q_rope,
                const void* k_rope, void* o, float* s, float* km, void* workspace,
                size_t workspace_bytes_, int64_t B, int64_t H, int64_t L, int DK, int DV, int dtype,
                int flags, float scale, float eps, void* stream) {
  const char* what = "fbla_la_fwd";
  int rc = check_dims(what, B, H, L, DK, DV, dtype, flags);
  if (rc != kOk) return rc;
  if (flags & kDefaultScale) {
    set_error("%s: FBLA_DEFAULT_SCALE is only valid for the packed entry points", what);
    return kErrBadArg;
  }
  if (!q || !k || !v || !o || !s || ((flags & kNormalize) && !km) ||
      ((flags & kDecoupled) && (!q_rope || !k_rope))) {
    if (B * H * L != 0) {
      set_error("%s: null tensor pointer", what);
      return kErrBadArg;
    }
  }
  Prob p = make_prob(nullptr, B, H, L, B * L, DK, DV, flags, scale, eps);
  FwdArgs a{q, k, v, q_rope, k_rope, o, s, km, workspace, workspace_bytes_};
  return run_fwd(what, p, dtype, a, (hipStream_t)stream);
}

int fbla_la_bwd(const void* q, const void* k, const void* v, const void* q_rope,
                const void* k_rope, const void* dout, const float* s, const float* km, void* dq,
                void* dk, void* dv, void* dq_rope, void* dk_rope, void* workspace,
                size_t workspace_bytes_, int64_t B, int64_t H, int64_t L, int DK, int DV, int dtype,
                int flags, float scale, float eps, void* stream) {
  const char* what = "fbla_la_bwd";
  int rc = check_dims(what, B, H, L, DK, DV, dtype, flags);
  if (rc != kOk) return rc;
  if (flags & kDefaultScale) {
    set_error("%s: FBLA_DEFAULT_SCALE is only valid for the packed entry points", what);
    return kErrBadArg;
  }
  const bool dec = flags & kDecoupled;
  if (B * H * L != 0 &&
      (!q || !v || !dout || !s || !dq || !dk || !dv || (!dec && !k) || ((flags & kNormalize) && !km) ||
       (dec && (!q_rope || !k_rope || !dq_rope || !dk_rope)))) {
    set_error("%s: null tensor pointer", what);
    return kErrBadArg;
  }
  Prob p = make_prob(nullptr, B, H, L, B * L, DK, DV, flags, scale, eps);
  BwdArgs a{q, k, v, q_rope, k_rope, dout, s, km, dq, dk, dv, dq_rope, dk_rope, workspace,
            workspace_bytes_};
  return run_bwd(what, p, dtype, a, (hipStream_t)stream);
}

// ---- the entry point that allocates nothing ------------------------------------------------
// Workspace of fbla_la_fwd_static: a fixed array in the library's device image.  Every GPU the
// library runs on holds its own copy at its own address until the process ends; host code may
// only use the address hipGetSymbolAddress returns for the current device, never the array's
// name (which is a host-side stand-in).
static constexpr size_t kStaticScratchBytes = (size_t)FBLA_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

static constexpr int kMaxDevices = 64;
static std::atomic<void*> g_scratch_ptr[kMaxDevices];  // zero-initialised: not looked up yet
static std::mutex g_scratch_mutex;

// Device address of `scratch` on the current device (looked up once per device), or null with
// the error text set.
static void* static_scratch(const char* what) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    set_error("%s: cannot identify the current device (%s)", what,
              e != hipSuccess ? hipGetErrorString(e) : "device index out of range");
    return nullptr;
  }
  void* ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (ptr) return ptr;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  ptr = g_scratch_ptr[dev].load(std::memory_order_relaxed);
  if (ptr) return ptr;
  e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
  if (e != hipSuccess || !ptr) {
    set_error("%s: hipGetSymbolAddress(scratch) failed on device %d: %s", what, dev, hipGetErrorString(e));
    return nullptr;
  }
  g_scratch_ptr[dev].store(ptr, std::memory_order_release);
  return ptr;
}

size_t fbla_static_scratch_bytes(void) { return kStaticScratchBytes; }

int fbla_la_fwd_static(const void* q, const void* k, const void* v, const void* q_rope, const void* k_rope,
                       void* o, float* s, float* km, int64_t B, int64_t H, int64_t L, int DK, int DV,
                       int dtype, int flags, float scale, float eps, void* stream) {
  const char* what = "fbla_la_fwd_static";
  int rc = check_dims(what, B, H, L, DK, DV, dtype, flags);
  if (rc != kOk) return rc;
  if (flags & kDefaultScale) {
    set_error("%s: FBLA_DEFAULT_SCALE is only valid for the packed entry points", what);
    return kErrBadArg;
  }
  if (B * H * L == 0) return kOk;
  if (!q || !k || !v || !o || !s || ((flags & kNormalize) && !km) ||
      ((flags & kDecoupled) && (!q_rope || !k_rope))) {
    set_error("%s: null tensor pointer", what);
    return kErrBadArg;
  }
  Prob p = make_prob(nullptr, B, H, L, B * L, DK, DV, flags, scale, eps);
  const size_t need = workspace_bytes(p, dtype, 0);
  if (need > kStaticScratchBytes) {
    set_error("%s: this problem needs %zu bytes of workspace, the built-in scratch holds %zu; "
              "use fbla_la_fwd with a caller-provided workspace", what, need, kStaticScratchBytes);
    return kErrWorkspace;
  }
  void* ws = static_scratch(what);
  if (!ws) return kErrLaunch;
  // Every partial the reductions read is written earlier in the same call, so nothing in the
  // scratch has to start at zero.
  FwdArgs a{q, k, v, q_rope, k_rope, o, s, km, ws, kStaticScratchBytes};
  return run_fwd(what, p, dtype, a, (hipStream_t)stream);
}

// ---- two queries on shared keys and values ---------------------------------------------------
size_t fbla_la_pair_workspace_bytes(int pass, int64_t B, int64_t H, int64_t L, int DK, int DV, int dtype) {
  if (check_dims("fbla_la_pair_workspace_bytes", B, H, L, DK, DV, dtype, kNormalize) != kOk) return 0;
  Prob p = make_prob(nullptr, B, H, L, B * L, DK, DV, kNormalize, 1.f, 0.f);
  if (!plan::pair_supported(p, dtype)) return 0;
  return pass == 0 ? plan::pair_fwd_workspace_bytes(p, dtype) : plan::pair_bwd_workspace_bytes(p, dtype);
}

int fbla_la_pair_fwd(const void* q1, const void* q2, const void* k, const void* v, void* o1, void* o2, float* s,
                     float* km, void* workspace, size_t workspace_bytes_, int64_t B, int64_t H, int64_t L, int DK,
                     int DV, int dtype, float scale, float eps, void* stream) {
  const char* what = "fbla_la_pair_fwd";
  int rc = check_dims(what, B, H, L, DK, DV, dtype, kNormalize);
  if (rc != kOk) return rc;
  if (B * H * L == 0) return kOk;
  if (!q1 || !q2 || !k || !v || !o1 || !o2 || !s || !km) {
    set_error("%s: null tensor pointer", what);
    return kErrBadArg;
  }
  if (check_aligned(what, {q1, q2, k, v, o1, o2, s, km, workspace}) != kOk) return kErrBadArg;
  Prob p = make_prob(nullptr, B, H, L, B * L, DK, DV, kNormalize, scale, eps);
  if (!plan::pair_supported(p, dtype)) {
    set_error("%s: needs dense fp16 / bf16 tensors with DK, DV/2 multiples of 8 (got DK=%d DV=%d dtype=%d)", what, DK,
              DV, dtype);
    return kErrUnsupported;
  }
  const size_t need = plan::pair_fwd_workspace_bytes(p, dtype);
  if (workspace_bytes_ < need || !workspace) {
    set_error("%s: workspace too small (%zu < %zu bytes)", what, workspace_bytes_, need);
    return kErrWorkspace;
  }
  PairFwdArgs a{{q1, q2}, k, v, {o1, o2}, s, km, workspace, workspace_bytes_};
  rc = plan::pair_forward(p, dtype, a, (hipStream_t)stream);
  return rc != kOk ? rc : check_launch(what);
}

int fbla_la_pair_bwd(const void* q1, const void* q2, const void* k, const void* v, const void* dout1,
                     const void* dout2, const float* s, const float* km, void* dq1, void* dq2, void* dk, void* dv,
                     void* workspace, size_t workspace_bytes_, int64_t B, int64_t H, int64_t L, int DK, int DV,
                     int dtype, float scale, float eps, void* stream) {
  const char* what = "fbla_la_pair_bwd";
  int rc = check_dims(what, B, H, L, DK, DV, dtype, kNormalize);
  if (rc != kOk) return rc;
  if (B * H * L == 0) return kOk;
  if (!q1 || !q2 || !k || !v || !dout1 || !dout2 || !s || !km || !dq1 || !dq2 || !dk || !dv) {
    set_error("%s: null tensor pointer", what);
    return kErrBadArg;
  }
  if (check_aligned(what, {q1, q2, k, v, dout1, dout2, s, km, dq1, dq2, dk, dv, workspace}) != kOk) return kErrBadArg;
  Prob p = make_prob(nullptr, B, H, L, B * L, DK, DV, kNormalize, scale, eps);
  if (!plan::pair_supported(p, dtype)) {
    set_error("%s: needs dense fp16 / bf16 tensors with DK, DV/2 multiples of 8 (got DK=%d DV=%d dtype=%d)", what, DK,
              DV, dtype);
    return kErrUnsupported;
  }
  const size_t need = plan::pair_bwd_workspace_bytes(p, dtype);
  if (workspace_bytes_ < need || !workspace) {
    set_error("%s: workspace too small (%zu < %zu bytes)", what, workspace_bytes_, need);
    return kErrWorkspace;
  }
  PairBwdArgs a{{q1, q2}, k, v, {dout1, dout2}, s, km, {dq1, dq2}, dk, dv, workspace, workspace_bytes_};
  rc = plan::pair_backward(p, dtype, a, (hipStream_t)stream);
  return rc != kOk ? rc : check_launch(what);
}

static int check_cross(const char* what, int64_t Lk, int flags) {
  if (Lk <= 0 || Lk > 0x7fffffffLL / 2) {
    set_error("%s: the number of keys must be positive and fit 32-bit indexing, got %lld", what, (long long)Lk);
    return kErrBadArg;
  }
  if (flags & kDefaultScale) {
    set_error("%s: FBLA_DEFAULT_SCALE is only valid for the packed entry points", what);
    return kErrBadArg;
  }
  return kOk;
}

size_t fbla_la_cross_workspace_bytes(int pass, int64_t B, int64_t H, int64_t Lq, int64_t Lk, int DK, int DV,
                                     int dtype, int flags) {
  const char* what = "fbla_la_cross_workspace_bytes";
  if (check_dims(what, B, H, Lq, DK, DV, dtype, flags) != kOk || check_cross(what, Lk, flags) != kOk) return 0;
  Prob p = make_prob(nullptr, B, H, Lq, B * Lq, DK, DV, flags, 1.f, 0.f);
  p.Lk = (int)Lk;
  return workspace_bytes(p, dtype, pass);
}

static int cross_fwd(const char* what, const void* q, const void* k, const void* v, const void* q_rope,
                     const void* k_rope, void* o, float* s, float* km, void* workspace, size_t workspace_bytes_,
                     int64_t B, int64_t H, int64_t Lq, int64_t Lk, int DK, int DV, int dtype, int flags, float scale,
                     float eps, void* stream) {
  int rc = check_dims(what, B, H, Lq, DK, DV, dtype, flags);
  if (rc == kOk) rc = check_cross(what, Lk, flags);
  if (rc != kOk) return rc;
  if (B * H > 0 && Lq > 0 &&
      (!q || !k || !v || !o || !s || ((flags & kNormalize) && !km) || ((flags & kDecoupled) && (!q_rope || !k_rope)))) {
    set_error("%s: null tensor pointer", what);
    return kErrBadArg;
  }
  Prob p = make_prob(nullptr, B, H, Lq, B * Lq, DK, DV, flags, scale, eps);
  p.Lk = (int)Lk;
  FwdArgs a{q, k, v, q_rope, k_rope, o, s, km, workspace, workspace_bytes_};
  return run_fwd(what, p, dtype, a, (hipStream_t)stream);
}

int fbla_la_cross_fwd(const void* q, const void* k, const void* v, void* o, float* s, float* km,
                      void* workspace, size_t workspace_bytes_, int64_t B, int64_t H, int64_t Lq, int64_t Lk,
                      int DK, int DV, int dtype, int flags, float scale, float eps, void* stream) {
  if (flags & kDecoupled) {
    set_error("fbla_la_cross_fwd: the decoupled operator takes its rotary rows through fbla_decoupled_cross_fwd");
    return kErrBadArg;
  }
  return cross_fwd("fbla_la_cross_fwd", q, k, v, nullptr, nullptr, o, s, km, workspace, workspace_bytes_, B, H, Lq, Lk,
                   DK, DV, dtype, flags, scale, eps, stream);
}

int fbla_decoupled_cross_fwd(const void* q, const void* k, const void* q_rope, const void* k_rope, const void* v,
                             void* o, float* s, float* km, void* workspace, size_t workspace_bytes_, int64_t B,
                             int64_t H, int64_t Lq, int64_t Lk, int DK, int DV, int dtype, float scale, float eps,
                             void* stream) {
  return cross_fwd("fbla_decoupled_cross_fwd", q, k, v, q_rope, k_rope, o, s, km, workspace, workspace_bytes_, B, H, Lq,
                   Lk, DK, DV, dtype, kNormalize | kDecoupled, scale, eps, stream);
}

static int cross_bwd(const char* what, const void* q, const void* k, const void* v, const void* q_rope,
                     const void* k_rope, const void* dout, const float* s, const float* km, void* dq, void* dk,
                     void* dv, void* dq_rope, void* dk_rope, void* workspace, size_t workspace_bytes_, int64_t B,
                     int64_t H, int64_t Lq, int64_t Lk, int DK, int DV, int dtype, int flags, float scale, float eps,
                     void* stream) {
  int rc = check_dims(what, B, H, Lq, DK, DV, dtype, flags);
  if (rc == kOk) rc = check_cross(what, Lk, flags);
  if (rc != kOk) return rc;
  const bool dec = flags & kDecoupled;
  if (B * H > 0 && Lq > 0 &&
      (!q || !v || !dout || !s || ((flags & kNormalize) && !km) || !dq || !dk || !dv || (!dec && !k) ||
       (dec && (!q_rope || !k_rope || !dq_rope || !dk_rope)))) {
    set_error("%s: null tensor pointer", what);
    return kErrBadArg;
  }
  Prob p = make_prob(nullptr, B, H, Lq, B * Lq, DK, DV, flags, scale, eps);
  p.Lk = (int)Lk;
  BwdArgs a{q, k, v, q_rope, k_rope, dout, s, km, dq, dk, dv, dq_rope, dk_rope, workspace, workspace_bytes_};
  return run_bwd(what, p, dtype, a, (hipStream_t)stream);
}

int fbla_la_cross_bwd(const void* q, const void* k, const void* v, const void* dout, const float* s,
                      const float* km, void* dq, void* dk, void* dv, void* workspace, size_t workspace_bytes_,
                      int64_t B, int64_t H, int64_t Lq, int64_t Lk, int DK, int DV, int dtype, int flags,
                      float scale, float eps, void* stream) {
  if (flags & kDecoupled) {
    set_error("fbla_la_cross_bwd: the decoupled operator takes its rotary rows through fbla_decoupled_cross_bwd");
    return kErrBadArg;
  }
  return cross_bwd("fbla_la_cross_bwd", q, k, v, nullptr, nullptr, dout, s, km, dq, dk, dv, nullptr, nullptr, workspace,
                   workspace_bytes_, B, H, Lq, Lk, DK, DV, dtype, flags, scale, eps, stream);
}

int fbla_decoupled_cross_bwd(const void* q, const void* k, const void* q_rope, const void* k_rope, const void* v,
                             const void* dout, const float* s, const float* km, void* dq, void* dk, void* dq_rope,
                             void* dk_rope, void* dv, void* workspace, size_t workspace_bytes_, int64_t B, int64_t H,
                             int64_t Lq, int64_t Lk, int DK, int DV, int dtype, float scale, float eps, void* stream) {
  return cross_bwd("fbla_decoupled_cross_bwd", q, k, v, q_rope, k_rope, dout, s, km, dq, dk, dv, dq_rope, dk_rope,
                   workspace, workspace_bytes_, B, H, Lq, Lk, DK, DV, dtype, kNormalize | kDecoupled, scale, eps, stream);
}

size_t fbla_varlen_workspace_bytes(int pass, int64_t total_tokens, int64_t N, int64_t H,
                                   int64_t max_seqlen, int DK, int DV, int dtype, int flags) {
  if (check_dims("fbla_varlen_workspace_bytes", N, H, max_seqlen, DK, DV, dtype, flags) != kOk)
    return 0;
  static const int32_t dummy = 0;
  Prob p = make_prob(&dummy, N, H, max_seqlen, total_tokens, DK, DV, flags, 1.f, 0.f);
  return workspace_bytes(p, dtype, pass);
}

int fbla_varlen_fwd(const void* q, const void* k, const void* v, const int32_t* cu_seqlens,
                    void* o, float* s, float* km, void* workspace, size_t workspace_bytes_,
                    int64_t total_tokens, int64_t N, int64_t H, int64_t max_seqlen, int DK, int DV,
                    int dtype, int flags, float scale, float eps, void* stream) {
  const char* what = "fbla_varlen_fwd";
  int rc = check_dims(what, N, H, max_seqlen, DK, DV, dtype, flags);
  if (rc != kOk) return rc;
  if ((flags & kDecoupled) || !(flags & kNormalize)) {
    set_error("%s: only the normalised, non-decoupled operator has a packed form", what);
    return kErrUnsupported;
  }
  if (total_tokens == 0 || N == 0) return kOk;
  if (!q || !k || !v || !o || !s || !km || !cu_seqlens) {
    set_error("%s: null tensor pointer", what);
    return kErrBadArg;
  }
  Prob p = make_prob(cu_seqlens, N, H, max_seqlen, total_tokens, DK, DV, flags, scale, eps);
  FwdArgs a{q, k, v, nullptr, nullptr, o, s, km, workspace, workspace_bytes_};
  return run_fwd(what, p, dtype, a, (hipStream_t)stream);
}

int fbla_varlen_bwd(const void* q, const void* k, const void* v, const int32_t* cu_seqlens,
                    const void* dout, const float* s, const float* km, void* dq, void* dk, void* dv,
                    void* workspace, size_t workspace_bytes_, int64_t total_tokens, int64_t N,
                    int64_t H, int64_t max_seqlen, int DK, int DV, int dtype, int flags,
                    float scale, float eps, void* stream) {
  const char* what = "fbla_varlen_bwd";
  int rc = check_dims(what, N, H, max_seqlen, DK, DV, dtype, flags);
  if (rc != kOk) return rc;
  if ((flags & kDecoupled) || !(flags & kNormalize)) {
    set_error("%s: only the normalised, non-decoupled operator has a packed form", what);
    return kErrUnsupported;
  }
  if (total_tokens == 0 || N == 0) return kOk;
  if (!q || !k || !v || !dout || !s || !km || !dq || !dk || !dv || !cu_seqlens) {
    set_error("%s: null tensor pointer", what);
    return kErrBadArg;
  }
  Prob p = make_prob(cu_seqlens, N, H, max_seqlen, total_tokens, DK, DV, flags, scale, eps);
  BwdArgs a{q, k, v, nullptr, nullptr, dout, s, km, dq, dk, dv, nullptr, nullptr, workspace,
            workspace_bytes_};
  return run_bwd(what, p, dtype, a, (hipStream_t)stream);
}

size_t fbla_chunk_reduce_workspace_bytes(int64_t BH, int64_t T, int K, int V, int chunk, int dtype,
                                         int with_norm) {
  if (check_dims("fbla_chunk_reduce_workspace_bytes", BH, 1, T, K, V, dtype, 0) != kOk || chunk < 1)
    return 0;
  return piecewise::chunk_reduce_workspace_bytes(BH, T, K, V, chunk, dtype, with_norm != 0);
}

int fbla_chunk_reduce(const void* q, const void* k, const void* v, float* qc, float* kc, float* vc,
                      float* h, float* h_norm, void* workspace, size_t workspace_bytes_, int64_t BH,
                      int64_t T, int K, int V, int chunk, float p_norm, int dtype, void* stream) {
  const char* what = "fbla_chunk_reduce";
  int rc = check_dims(what, BH, 1, T, K, V, dtype, 0);
  if (rc != kOk) return rc;
  if (chunk < 1 || (h_norm && !(p_norm > 0.f))) {
    set_error("%s: chunk must be positive and the norm order > 0", what);
    return kErrBadArg;
  }
  if (BH == 0 || T == 0) return kOk;
  if (!q || !k || !v || !qc || !kc || !vc || !h) {
    set_error("%s: null tensor pointer", what);
    return kErrBadArg;
  }
  const size_t need = piecewise::chunk_reduce_workspace_bytes(BH, T, K, V, chunk, dtype, h_norm != nullptr);
  if (workspace_bytes_ < need || !workspace) {
    set_error("%s: workspace too small (%zu < %zu bytes)", what, workspace_bytes_, need);
    return kErrWorkspace;
  }
  rc = piecewise::chunk_reduce(q, k, v, qc, kc, vc, h, h_norm, workspace, BH, T, K, V, chunk, p_norm,
                               dtype, (hipStream_t)stream);
  if (rc != kOk) return rc;
  return check_launch(what);
}

// 16-bit inputs, blocks of a multiple of 64 tokens, head dims other than 64 / 128: the matrix-core kernel runs on copies
// widened with zeros to 64 / 128 (zero key features leave every score as it is, zero value columns give
// zero output columns, which are dropped again) instead of the shape-generic kernel, which is about ten
// times slower.  q | k | v | o | kc | vc | h (widened) | the kernel's own workspace
static int pw_wide(int d) { return d <= 64 ? 64 : 128; }
static bool pw_widen(int K, int V, int block, int dtype) {
  return (dtype == kF16 || dtype == kBF16) && piecewise::attention_supported(64, 64, block, dtype) && K <= 128 &&
         V <= 128 &&
         !piecewise::attention_supported(K, V, block, dtype);
}
static size_t pw_widened_bytes(int64_t BH, int64_t T, int K, int V, int block) {
  const int Kw = pw_wide(K), Vw = pw_wide(V);
  const int64_t NT = (T + block - 1) / block;
  return 2 * align_up((size_t)BH * T * Kw * 2, 256) + 2 * align_up((size_t)BH * T * Vw * 2, 256) +
         align_up((size_t)BH * NT * Kw * 4, 256) + align_up((size_t)BH * NT * Vw * 4, 256) +
         align_up((size_t)BH * Kw * Vw * 4, 256) + piecewise::attention_workspace_bytes(BH, T, Kw, Vw, block);
}

size_t fbla_piecewise_workspace_bytes(int64_t BH, int64_t T, int K, int V, int block, int dtype) {
  if (check_dims("fbla_piecewise_workspace_bytes", BH, 1, T, K, V, dtype, 0) != kOk) return 0;
  if (piecewise::attention_supported(K, V, block, dtype)) return piecewise::attention_workspace_bytes(BH, T, K, V, block);
  if (pw_widen(K, V, block, dtype)) return pw_widened_bytes(BH, T, K, V, block);
  // the shape-generic kernel needs no workspace; a token size keeps "0 = not supported"
  return piecewise::attention_generic_supported(T, K, V, block, dtype) ? 256 : 0;
}

int fbla_piecewise_fwd(const void* q, const void* k, const void* v, const float* kc, const float* vc,
                       const float* h, const int32_t* indices, void* o, void* workspace,
                       size_t workspace_bytes_, int64_t BH, int64_t T, int K, int V, int block, int NS,
                       float scale, int dtype, void* stream) {
  const char* what = "fbla_piecewise_fwd";
  int rc = check_dims(what, BH, 1, T, K, V, dtype, 0);
  if (rc != kOk) return rc;
  const bool widen = pw_widen(K, V, block, dtype);
  const bool fast = widen || piecewise::attention_supported(K, V, block, dtype);
  if (!fast && !piecewise::attention_generic_supported(T, K, V, block, dtype)) {
    set_error("%s: needs head dims in [1,128], a positive block size and block flags that fit LDS "
              "(got K=%d V=%d block=%d dtype=%d T=%lld)", what, K, V, block, dtype, (long long)T);
    return kErrUnsupported;
  }
  const int64_t NT = (T + block - 1) / block;
  if (NS < 1 || NS > NT) {
    set_error("%s: the number of selected blocks must be in [1, %lld], got %d", what, (long long)NT, NS);
    return kErrBadArg;
  }
  if (BH == 0 || T == 0) return kOk;
  if (!q || !k || !v || !kc || !vc || !h || !indices || !o) {
    set_error("%s: null tensor pointer", what);
    return kErrBadArg;
  }
  if (!fast) {
    rc = piecewise::attention_generic(q, k, v, kc, vc, h, indices, o, BH, T, K, V, block, NS, scale, dtype,
                                      (hipStream_t)stream);
    if (rc != kOk) return rc;
    return check_launch(what);
  }
  const size_t need = widen ? pw_widened_bytes(BH, T, K, V, block) : piecewise::attention_workspace_bytes(BH, T, K, V, block);
  if (workspace_bytes_ < need || !workspace) {
    set_error("%s: workspace too small (%zu < %zu bytes)", what, workspace_bytes_, need);
    return kErrWorkspace;
  }
  if (widen) {
    hipStream_t st = (hipStream_t)stream;
    const int Kw = pw_wide(K), Vw = pw_wide(V);
    char* ws = (char*)workspace;
    auto take = [&](size_t bytes) { void* r = ws; ws += align_up(bytes, 256); return r; };
    void* qw = take((size_t)BH * T * Kw * 2);
    void* kw = take((size_t)BH * T * Kw * 2);
    void* vw = take((size_t)BH * T * Vw * 2);
    void* ow = take((size_t)BH * T * Vw * 2);
    float* kcw = (float*)take((size_t)BH * NT * Kw * 4);
    float* vcw = (float*)take((size_t)BH * NT * Vw * 4);
    float* hw = (float*)take((size_t)BH * Kw * Vw * 4);
    generic::resize_matrices(q, BH * T, K, qw, BH * T, Kw, 1, 2, st);
    generic::resize_matrices(k, BH * T, K, kw, BH * T, Kw, 1, 2, st);
    generic::resize_matrices(v, BH * T, V, vw, BH * T, Vw, 1, 2, st);
    generic::resize_matrices(kc, BH * NT, K, kcw, BH * NT, Kw, 1, 4, st);
    generic::resize_matrices(vc, BH * NT, V, vcw, BH * NT, Vw, 1, 4, st);
    generic::resize_matrices(h, K, V, hw, Kw, Vw, BH, 4, st);
    rc = piecewise::attention(qw, kw, vw, kcw, vcw, hw, indices, ow, ws, BH, T, Kw, Vw, block, NS, scale, dtype, st);
    if (rc != kOk) return rc;
    generic::resize_matrices(ow, BH * T, Vw, o, BH * T, V, 1, 2, st);
    return check_launch(what);
  }
  rc = piecewise::attention(q, k, v, kc, vc, h, indices, o, workspace, BH, T, K, V, block, NS, scale, dtype,
                            (hipStream_t)stream);
  if (rc != kOk) return rc;
  return check_launch(what);
}

int fbla_select_blocks(const float* qc, const float* kc, const float* bias, int32_t* indices,
                       int64_t BH, int64_t NT, int K, int NS, float scale, void* stream) {
  const char* what = "fbla_select_blocks";
  if (BH < 0 || NT < 0 || NT > 0x7fffffffLL / 64) {
    set_error("%s: bad sizes BH=%lld NT=%lld", what, (long long)BH, (long long)NT);
    return kErrBadArg;
  }
  if (BH == 0 || NT == 0) return kOk;
  if (NS < 1 || NS > NT) {
    set_error("%s: the number of selected blocks must be in [1, %lld], got %d", what, (long long)NT, NS);
    return kErrBadArg;
  }
  if (!piecewise::select_blocks_supported((int)NT, K)) {
    set_error("%s: needs K in [1,128] and a score row that fits LDS (got K=%d NT=%lld)", what, K,
              (long long)NT);
    return kErrUnsupported;
  }
  if (!qc || !kc || !indices) {
    set_error("%s: null tensor pointer", what);
    return kErrBadArg;
  }
  int rc = piecewise::select_blocks(qc, kc, bias, indices, BH, (int)NT, K, NS, scale, (hipStream_t)stream);
  if (rc != kOk) return rc;
  return check_launch(what);
}

int fbla_elu1_fwd(const void* x0, void* y0, int64_t n0, const void* x1, void* y1, int64_t n1, int dtype,
                  void* stream) {
  const char* what = "fbla_elu1_fwd";
  if (n0 < 0 || n1 < 0 || (dtype != kF16 && dtype != kBF16 && dtype != kF32)) {
    set_error("%s: bad sizes or dtype (n0=%lld n1=%lld dtype=%d)", what, (long long)n0, (long long)n1, dtype);
    return kErrBadArg;
  }
  if (n0 == 0 && n1 == 0) return kOk;
  if ((n0 > 0 && (!x0 || !y0)) || (n1 > 0 && (!x1 || !y1))) {
    set_error("%s: null tensor pointer", what);
    return kErrBadArg;
  }
  if (check_aligned(what, {n0 > 0 ? x0 : nullptr, n0 > 0 ? y0 : nullptr, n1 > 0 ? x1 : nullptr,
                           n1 > 0 ? y1 : nullptr}) != kOk)
    return kErrBadArg;
  feature::elu1_fwd(x0, y0, n0, x1, y1, n1, dtype, (hipStream_t)stream);
  return check_launch(what);
}

int fbla_elu1_bwd(const void* x, const void* dy, void* dx, int64_t n, int dtype, void* stream) {
  const char* what = "fbla_elu1_bwd";
  if (n < 0 || (dtype != kF16 && dtype != kBF16 && dtype != kF32)) {
    set_error("%s: bad size or dtype (n=%lld dtype=%d)", what, (long long)n, dtype);
    return kErrBadArg;
  }
  if (n == 0) return kOk;
  if (!x || !dy || !dx) {
    set_error("%s: null tensor pointer", what);
    return kErrBadArg;
  }
  if (check_aligned(what, {x, dy, dx}) != kOk) return kErrBadArg;
  feature::elu1_bwd(x, dy, dx, n, dtype, (hipStream_t)stream);
  return check_launch(what);
}

}  // extern "C"
