// C ABI: jvpfa_fwd and the small query functions.
#include <hip/hip_runtime.h>
#include <stddef.h>

#include "api_common.hpp"
#include "split.hpp"

namespace jvpfa {
#define JVPFA_DECL(name) int name(const FwdParams &, bool, int, hipStream_t);
JVPFA_DECL(fwd_bf16_32) JVPFA_DECL(fwd_bf16_64) JVPFA_DECL(fwd_bf16_128) JVPFA_DECL(fwd_bf16_256)
JVPFA_DECL(fwd_fp16_32) JVPFA_DECL(fwd_fp16_64) JVPFA_DECL(fwd_fp16_128) JVPFA_DECL(fwd_fp16_256)
JVPFA_DECL(fwd_fp32_32) JVPFA_DECL(fwd_fp32_64) JVPFA_DECL(fwd_fp32_128) JVPFA_DECL(fwd_fp32_256)
#undef JVPFA_DECL
typedef int (*fwd_launcher)(const FwdParams &, bool, int, hipStream_t);
static const fwd_launcher kFwd[12] = {fwd_bf16_32, fwd_bf16_64, fwd_bf16_128, fwd_bf16_256, fwd_fp16_32, fwd_fp16_64,
                                      fwd_fp16_128, fwd_fp16_256, fwd_fp32_32, fwd_fp32_64, fwd_fp32_128, fwd_fp32_256};
}  // namespace jvpfa

using namespace jvpfa;

extern "C" int jvpfa_fwd(const jvpfa_fwd_args *a, void *hip_stream) {
  if (!a) return JVPFA_E_NULL;
  if (a->struct_size != sizeof(jvpfa_fwd_args)) return JVPFA_E_ABI;
  int rc = check_problem(a->p);
  if (rc == JVPFA_OK) rc = check_kv_shape(a->p, a->Lk, a->Hk);
  if (rc != JVPFA_OK) return rc;
  if (!a->q || !a->k || !a->v || !a->o || !a->M) return JVPFA_E_NULL;
  const int ntan = (a->qt != nullptr) + (a->kt != nullptr) + (a->vt != nullptr);
  if (ntan != 0 && ntan != 3) return JVPFA_E_NULL;
  const bool dual = ntan == 3;
  if (dual && (!a->ot || !a->mu)) return JVPFA_E_NULL;
  const void *ptrs[] = {a->q, a->k, a->v, a->qt, a->kt, a->vt, a->o, a->ot};
  for (const void *ptr : ptrs)
    if (ptr && !aligned16(ptr)) return JVPFA_E_ALIGN;

  FwdParams p;
  p.pr = to_problem(a->p, a->key_limit, a->tiles_q, nullptr, a->Lk, a->Hk);
  p.q = a->q; p.k = a->k; p.v = a->v;
  p.qt = a->qt; p.kt = a->kt; p.vt = a->vt;
  p.o = a->o; p.ot = a->ot; p.M = a->M; p.mu = a->mu;
  if (a->split_workspace) {  // small grid: split the key tiles of every query block, if the workspace suffices
    const SplitPlan sp = fwd_split_plan(a->p, p.pr.Lk);
    if (sp.chunks > 1 && aligned16(a->split_workspace) &&
        a->split_workspace_bytes >= fwd_part_floats(sp.chunks, (long long)a->p.Z * a->p.H * a->p.L, a->p.D) * sizeof(float)) {
      p.pr.chunks = sp.chunks;
      p.pr.chunk_tiles = sp.chunk_tiles;
      p.pr.part = static_cast<float *>(a->split_workspace);
    }
  }
  return kFwd[slot(a->p)](p, dual, a->p.mask_kind, static_cast<hipStream_t>(hip_stream));
}

extern "C" size_t jvpfa_fwd_split_workspace_bytes(const jvpfa_problem *p, int32_t Lk) {
  if (!p || check_problem(*p) != JVPFA_OK) return 0;
  const SplitPlan sp = fwd_split_plan(*p, Lk > 0 ? Lk : p->L);
  return sp.chunks > 1 ? fwd_part_floats(sp.chunks, (long long)p->Z * p->H * p->L, p->D) * sizeof(float) : 0;
}

extern "C" int jvpfa_abi_version(void) { return JVPFA_ABI_VERSION; }

extern "C" const char *jvpfa_error_string(int status) {
  switch (status) {
    case JVPFA_OK: return "ok";
    case JVPFA_E_NULL: return "a required pointer is NULL";
    case JVPFA_E_SHAPE: return "unsupported shape (Z,H,L >= 1 and D in {32,64,128,256} and dropout_p in [0,1) required)";
    case JVPFA_E_DTYPE: return "dtype or mask kind out of range";
    case JVPFA_E_ALIGN: return "tensor pointer not 16-byte aligned";
    case JVPFA_E_CONFLICT: return "causal attention does not take a mask";
    case JVPFA_E_LAUNCH: return "HIP kernel launch failed";
    case JVPFA_E_SCRATCH: return "Z*H*L exceeds the rows of the library's static scratch (jvpfa_bwd_static_max_rows())";
    case JVPFA_E_ABI: return "struct_size does not match this library: caller and library were built from different headers";
  }
  return "unknown status";
}
