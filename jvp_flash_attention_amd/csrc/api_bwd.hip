// C ABI: jvpfa_bwd and its workspace size.
#include <hip/hip_runtime.h>
#include <stddef.h>

#include "api_common.hpp"

namespace jvpfa {
#define JVPFA_DECL(name) int name(const BwdParams &, int, bool, bool, hipStream_t);
JVPFA_DECL(bwd_bf16_32) JVPFA_DECL(bwd_bf16_64) JVPFA_DECL(bwd_bf16_128) JVPFA_DECL(bwd_bf16_256)
JVPFA_DECL(bwd_fp16_32) JVPFA_DECL(bwd_fp16_64) JVPFA_DECL(bwd_fp16_128) JVPFA_DECL(bwd_fp16_256)
JVPFA_DECL(bwd_fp32_32) JVPFA_DECL(bwd_fp32_64) JVPFA_DECL(bwd_fp32_128)
#undef JVPFA_DECL
typedef int (*bwd_launcher)(const BwdParams &, int, bool, bool, hipStream_t);
static const bwd_launcher kBwd[12] = {bwd_bf16_32, bwd_bf16_64, bwd_bf16_128, bwd_bf16_256, bwd_fp16_32, bwd_fp16_64,
                                      bwd_fp16_128, bwd_fp16_256, bwd_fp32_32, bwd_fp32_64, bwd_fp32_128, nullptr};

// Each row statistic is padded to a multiple of 4 floats so the three arrays stay 16-byte aligned.
static inline size_t stat_floats(int Z, int H, int L) { return (((size_t)Z * H * L) + 3) & ~(size_t)3; }
}  // namespace jvpfa

using namespace jvpfa;

extern "C" size_t jvpfa_bwd_workspace_bytes(int32_t Z, int32_t H, int32_t L) {
  if (Z < 1 || H < 1 || L < 1) return 0;
  return 3 * stat_floats(Z, H, L) * sizeof(float);
}

extern "C" int jvpfa_bwd(const jvpfa_bwd_args *a, void *hip_stream) {
  if (!a) return JVPFA_E_NULL;
  if (a->struct_size != sizeof(jvpfa_bwd_args)) return JVPFA_E_ABI;
  if ((a->tiles_q != nullptr) != (a->tiles_k != nullptr)) return JVPFA_E_NULL;
  int rc = check_problem(a->p);
  if (rc == JVPFA_OK) rc = check_kv_shape(a->p, a->Lk, a->Hk);
  if (rc != JVPFA_OK) return rc;
  if (!a->q || !a->k || !a->v || !a->o || !a->M || !a->dq || !a->dk || !a->dv || !a->workspace)
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
                        a->gt, a->dq, a->dk, a->dv, a->dqt, a->dkt, a->dvt, a->workspace};
  for (const void *ptr : ptrs)
    if (ptr && !aligned16(ptr)) return JVPFA_E_ALIGN;

  BwdParams p;
  p.pr = to_problem(a->p, a->key_limit, a->tiles_q, a->tiles_k, a->Lk, a->Hk);
  p.q = a->q; p.k = a->k; p.v = a->v;
  p.qt = a->qt; p.kt = a->kt; p.vt = a->vt;
  p.o = a->o; p.ot = a->ot; p.M = a->M; p.mu = a->mu;
  p.go = a->go; p.gt = a->gt;
  p.dq = a->dq; p.dk = a->dk; p.dv = a->dv;
  p.dqt = a->dqt; p.dkt = a->dkt; p.dvt = a->dvt;
  const size_t n = stat_floats(a->p.Z, a->p.H, a->p.L);
  p.d1 = static_cast<float *>(a->workspace);
  p.a = p.d1 + n;
  p.d2 = p.a + n;
  return kBwd[slot(a->p)](p, a->p.mask_kind, dual, ntg == 3, static_cast<hipStream_t>(hip_stream));
}
