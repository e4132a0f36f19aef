// C ABI: jvpfa_bwd, its workspace size, and jvpfa_bwd_static (row statistics in the library's own
// static device array instead of a caller's workspace).
#include <hip/hip_runtime.h>
#include <stddef.h>

#include <atomic>
#include <mutex>

#include "api_common.hpp"

namespace jvpfa {
#define JVPFA_DECL(name) int name(const BwdParams &, int, bool, bool, hipStream_t);
JVPFA_DECL(bwd_bf16_32) JVPFA_DECL(bwd_bf16_64) JVPFA_DECL(bwd_bf16_128) JVPFA_DECL(bwd_bf16_256)
JVPFA_DECL(bwd_fp16_32) JVPFA_DECL(bwd_fp16_64) JVPFA_DECL(bwd_fp16_128) JVPFA_DECL(bwd_fp16_256)
JVPFA_DECL(bwd_fp32_32) JVPFA_DECL(bwd_fp32_64) JVPFA_DECL(bwd_fp32_128) JVPFA_DECL(bwd_fp32_256)
#undef JVPFA_DECL
typedef int (*bwd_launcher)(const BwdParams &, int, bool, bool, hipStream_t);
static const bwd_launcher kBwd[12] = {bwd_bf16_32, bwd_bf16_64, bwd_bf16_128, bwd_bf16_256, bwd_fp16_32, bwd_fp16_64,
                                      bwd_fp16_128, bwd_fp16_256, bwd_fp32_32, bwd_fp32_64, bwd_fp32_128, bwd_fp32_256};

// Each row statistic is padded to a multiple of 4 floats so the three arrays stay 16-byte aligned.
static inline size_t stat_floats(int Z, int H, int L) { return (((size_t)Z * H * L) + 3) & ~(size_t)3; }
}  // namespace jvpfa

using namespace jvpfa;

extern "C" size_t jvpfa_bwd_workspace_bytes(int32_t Z, int32_t H, int32_t L) {
  if (Z < 1 || H < 1 || L < 1) return 0;
  return 3 * stat_floats(Z, H, L) * sizeof(float);
}

// Everything jvpfa_bwd does, with the row statistics of the pre-pass in `workspace`.
static int bwd_impl(const jvpfa_bwd_args *a, void *workspace, void *hip_stream) {
  if (!a) return JVPFA_E_NULL;
  if (a->struct_size != sizeof(jvpfa_bwd_args)) return JVPFA_E_ABI;
  if ((a->tiles_q != nullptr) != (a->tiles_k != nullptr)) return JVPFA_E_NULL;
  int rc = check_problem(a->p);
  if (rc == JVPFA_OK) rc = check_kv_shape(a->p, a->Lk, a->Hk);
  if (rc != JVPFA_OK) return rc;
  if (!a->q || !a->k || !a->v || !a->o || !a->M || !a->dq || !a->dk || !a->dv || !workspace)
    return JVPFA_E_NULL;
  const bool dual = a->gt != nullptr;
  if (dual) {
    if (!a->qt || !a->kt || !a->vt || !a->ot || !a->mu) return JVPFA_E_NULL;
  } else if (!a->go) {
    return JVPFA_E_NULL;
  }
  const int ntg = (a->dqt != nullptr) + (a->dkt != nullptr) + (a->dvt != nullptr);
  if (ntg != 0 && (ntg != 3 || !dual)) return JVPFA_E_NULL;
  const void *ptrs[] = {a->q,  a->k,  a->v,  a->qt, a->kt, a->vt,  a->o,   a->ot,  a->go,
                        a->gt, a->dq, a->dk, a->dv, a->dqt, a->dkt, a->dvt, workspace};
  for (const void *ptr : ptrs)
    if (ptr && !aligned16(ptr)) return JVPFA_E_ALIGN;

  BwdParams p;
  if (a->mask_bits && (reinterpret_cast<uintptr_t>(a->mask_bits) & 7u)) return JVPFA_E_ALIGN;
  p.pr = to_problem(a->p, a->key_limit, a->tiles_q, a->tiles_k, a->Lk, a->Hk, a->mask_bits);
  p.q = a->q; p.k = a->k; p.v = a->v;
  p.qt = a->qt; p.kt = a->kt; p.vt = a->vt;
  p.o = a->o; p.ot = a->ot; p.M = a->M; p.mu = a->mu;
  p.go = a->go; p.gt = a->gt;
  p.dq = a->dq; p.dk = a->dk; p.dv = a->dv;
  p.dqt = a->dqt; p.dkt = a->dkt; p.dvt = a->dvt;
  const size_t n = stat_floats(a->p.Z, a->p.H, a->p.L);
  p.d1 = static_cast<float *>(workspace);
  p.a = p.d1 + n;
  p.d2 = p.a + n;
  return kBwd[slot(a->p)](p, a->p.mask_kind, dual, ntg == 3, static_cast<hipStream_t>(hip_stream));
}

extern "C" int jvpfa_bwd(const jvpfa_bwd_args *a, void *hip_stream) {
  return bwd_impl(a, a ? a->workspace : nullptr, hip_stream);
}

// ---- the variant that brings its own workspace -------------------------------------------------
// One array per GPU, held from the moment the library's code object is loaded there until the
// process ends.  In host code the array's name only stands for the symbol; the address the kernels
// get is looked up once per device and kept.
static __device__ __align__(256) float scratch[3 * (size_t)JVPFA_STATIC_ROWS];

namespace {
constexpr int MAX_DEVICES = 64;
std::atomic<float *> g_scratch_ptr[MAX_DEVICES];
std::mutex g_scratch_mutex;

// The address of `scratch` on the current device, or null (with *status set) when it cannot be had.
float *scratch_on_current_device(int *status) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) {
    *status = JVPFA_E_LAUNCH;
    return nullptr;
  }
  float *ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (ptr) return ptr;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  ptr = g_scratch_ptr[dev].load(std::memory_order_relaxed);
  if (!ptr) {
    void *sym = nullptr;
    if (hipGetSymbolAddress(&sym, HIP_SYMBOL(scratch)) != hipSuccess || !sym) {
      (void)hipGetLastError();
      *status = JVPFA_E_LAUNCH;
      return nullptr;
    }
    ptr = static_cast<float *>(sym);
    g_scratch_ptr[dev].store(ptr, std::memory_order_release);
  }
  return ptr;
}
}  // namespace

extern "C" size_t jvpfa_bwd_static_max_rows(void) { return (size_t)JVPFA_STATIC_ROWS; }

extern "C" int jvpfa_bwd_static(const jvpfa_bwd_args *a, void *hip_stream) {
  if (!a) return JVPFA_E_NULL;
  if (a->struct_size != sizeof(jvpfa_bwd_args)) return JVPFA_E_ABI;
  if (a->p.Z < 1 || a->p.H < 1 || a->p.L < 1) return JVPFA_E_SHAPE;
  // the three statistics, each padded to a multiple of 4 floats, must fit the array
  if (stat_floats(a->p.Z, a->p.H, a->p.L) > (size_t)JVPFA_STATIC_ROWS) return JVPFA_E_SCRATCH;
  int status = JVPFA_OK;
  float *ws = scratch_on_current_device(&status);
  if (!ws) return status;
  // Nothing in the array has to start at zero: the pre-pass writes every statistic of every row
  // before the dq and dk/dv kernels, later on the same stream, read it.
  return bwd_impl(a, ws, hip_stream);
}
