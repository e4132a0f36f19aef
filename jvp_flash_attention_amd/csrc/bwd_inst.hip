// One translation unit per (element type, head dim): compiled with
//   -DJVPFA_T=<__bf16|_Float16|float> -DJVPFA_D=<32|64|128|256> -DJVPFA_NAME=<symbol>
// and exporting  int JVPFA_NAME(const BwdParams&, int mask_kind, bool dual, bool tangent_grads,
// hipStream_t): pre-pass, then the dq and dk/dv kernels of every requested mode.
#include "bwd_kernel.hpp"
#include "bwd_kernel_v2.hpp"
#include "bwd_kernel_wide.hpp"
#include "launch.hpp"

namespace jvpfa {

template <typename T, int D, int MODE, int MASK>
static int launch_bwd_mode(const BwdParams &p, hipStream_t stream) {
  using Cfg = BwdCfg<T, D, MODE>;
  const int nb = (p.pr.L + BWD_BLK - 1) / BWD_BLK;
  const long long blocks = (long long)nb * p.pr.Z * p.pr.H;
  if (blocks > 0x7fffffffLL) return -2;
  // the dk/dv kernels run one workgroup per 128 keys of a key/value head (the same count as for dq
  // when k, v have q's shape)
  const long long kv_blocks = (long long)((p.pr.Lk + BWD_BLK - 1) / BWD_BLK) * p.pr.Z * p.pr.Hk;
  if (kv_blocks > 0x7fffffffLL) return -2;
  if (p.pr.drop_thr != 0) {
    // dropout: every element type takes the register-staged kernels, the one family that carries it
    if constexpr (D <= 128) {
      auto kq = bwd_dq_kernel<T, D, MODE, MASK, true>;
      auto kkv = bwd_dkdv_kernel<T, D, MODE, MASK, true>;
      int rc = allow_lds(reinterpret_cast<const void *>(kq), Cfg::DQ_LDS);
      if (rc == 0) rc = allow_lds(reinterpret_cast<const void *>(kkv), Cfg::DKV_LDS);
      if (rc != 0) return rc;
      hipLaunchKernelGGL(kkv, dim3((unsigned)kv_blocks), dim3(BWD_NT), Cfg::DKV_LDS, stream, p);
      hipLaunchKernelGGL(kq, dim3((unsigned)blocks), dim3(BWD_NT), Cfg::DQ_LDS, stream, p);
      return hipGetLastError() == hipSuccess ? 0 : -6;
    }
    return -2;
  }
  if constexpr (sizeof(T) == 2 && D <= 128) {  // direct-to-LDS, double-buffered kernels
   {
    using Cfg2 = Bwd2Cfg<T, D, MODE>;
    // gO may be absent only in the dual mode (loss depends on O' alone)
    const bool no_go = MODE == BWD_DUAL && p.go == nullptr;
    constexpr bool NG = MODE != BWD_DUAL;  // the GO template argument of the kernels without gO
    void (*kq)(const BwdParams), (*kkv)(const BwdParams);
    const bool grouped = p.pr.Hk != p.pr.H;  // a key/value head serves several query heads
    if constexpr (D == 64) {  // the register-capped twins: two workgroups per compute unit (D = 32 needs no cap for that)
      kq = no_go ? bwd2_dq_kernel_2wg<T, D, MODE, MASK, NG> : bwd2_dq_kernel_2wg<T, D, MODE, MASK, true>;
      if constexpr (MASK == MASK_NONE || MODE != BWD_DUAL) {
        if (grouped) kkv = no_go ? bwd2_dkdv_kernel_2wg<T, D, MODE, MASK, NG, true> : bwd2_dkdv_kernel_2wg<T, D, MODE, MASK, true, true>;
        else kkv = no_go ? bwd2_dkdv_kernel_2wg<T, D, MODE, MASK, NG> : bwd2_dkdv_kernel_2wg<T, D, MODE, MASK, true>;
      } else {  // the masked dual dk/dv kernel needs a few registers more than the cap leaves
        if (grouped) kkv = no_go ? bwd2_dkdv_kernel<T, D, MODE, MASK, NG, true> : bwd2_dkdv_kernel<T, D, MODE, MASK, true, true>;
        else kkv = no_go ? bwd2_dkdv_kernel<T, D, MODE, MASK, NG> : bwd2_dkdv_kernel<T, D, MODE, MASK, true>;
      }
    } else {
      kq = no_go ? bwd2_dq_kernel<T, D, MODE, MASK, NG> : bwd2_dq_kernel<T, D, MODE, MASK, true>;
      if (grouped) kkv = no_go ? bwd2_dkdv_kernel<T, D, MODE, MASK, NG, true> : bwd2_dkdv_kernel<T, D, MODE, MASK, true, true>;
      else kkv = no_go ? bwd2_dkdv_kernel<T, D, MODE, MASK, NG> : bwd2_dkdv_kernel<T, D, MODE, MASK, true>;
    }
    int rc = allow_lds(reinterpret_cast<const void *>(kq), Cfg2::DQ_LDS);
    if (rc == 0) rc = allow_lds(reinterpret_cast<const void *>(kkv), Cfg2::DKV_LDS);
    if (rc != 0) return rc;
    hipLaunchKernelGGL(kkv, dim3((unsigned)kv_blocks), dim3(Cfg2::NT), Cfg2::DKV_LDS, stream, p);
    hipLaunchKernelGGL(kq, dim3((unsigned)blocks), dim3(Cfg2::NT), Cfg2::DQ_LDS, stream, p);
    return hipGetLastError() == hipSuccess ? 0 : -6;
   }
  } else if constexpr (sizeof(T) == 2 && D == 256) {
    // dq: two workgroups per query block, each with 128 of its columns, on the direct-to-LDS pipeline
    using CfgW = BwdWideCfg<T, D, 128, MODE>;
    const bool no_go = MODE == BWD_DUAL && p.go == nullptr;
    constexpr bool NG = MODE != BWD_DUAL;
    void (*kq)(const BwdParams) = no_go ? bwdw_dq_kernel<T, D, 128, MODE, MASK, NG> : bwdw_dq_kernel<T, D, 128, MODE, MASK, true>;
    if (blocks * CfgW::NS > 0x7fffffffLL) return -2;
    int rc = allow_lds(reinterpret_cast<const void *>(kq), CfgW::DQ_LDS);
    if (rc != 0) return rc;
    // dk/dv on the same pipeline: dV from K, K' alone, then dK in two column halves (dual); both in two
    // column halves (otherwise)
    using CfgK = BwdWideKvCfg<T, D, 128, MODE>;
    if (kv_blocks * CfgK::NS > 0x7fffffffLL) return -2;
    if constexpr (MODE == BWD_DUAL) {
      void (*kv)(const BwdParams) = no_go ? bwdw_dkdv_kernel<T, D, 128, MODE, MASK, NG, WIDE_DV>
                                          : bwdw_dkdv_kernel<T, D, 128, MODE, MASK, true, WIDE_DV>;
      void (*kk)(const BwdParams) = no_go ? bwdw_dkdv_kernel<T, D, 128, MODE, MASK, NG, WIDE_DK>
                                          : bwdw_dkdv_kernel<T, D, 128, MODE, MASK, true, WIDE_DK>;
      rc = allow_lds(reinterpret_cast<const void *>(kv), CfgK::DKV_LDS);
      if (rc == 0) rc = allow_lds(reinterpret_cast<const void *>(kk), CfgK::DKV_LDS);
      if (rc != 0) return rc;
      hipLaunchKernelGGL(kv, dim3((unsigned)kv_blocks), dim3(CfgK::NT), CfgK::DKV_LDS, stream, p);
      hipLaunchKernelGGL(kk, dim3((unsigned)(kv_blocks * CfgK::NS)), dim3(CfgK::NT), CfgK::DKV_LDS, stream, p);
    } else {
      auto kkv = bwdw_dkdv_kernel<T, D, 128, MODE, MASK, true, WIDE_BOTH>;
      rc = allow_lds(reinterpret_cast<const void *>(kkv), CfgK::DKV_LDS);
      if (rc != 0) return rc;
      hipLaunchKernelGGL(kkv, dim3((unsigned)(kv_blocks * CfgK::NS)), dim3(CfgK::NT), CfgK::DKV_LDS, stream, p);
    }
    hipLaunchKernelGGL(kq, dim3((unsigned)(blocks * CfgW::NS)), dim3(CfgW::NT), CfgW::DQ_LDS, stream, p);
    return hipGetLastError() == hipSuccess ? 0 : -6;
  } else {
    auto kq = bwd_dq_kernel<T, D, MODE, MASK>;
    auto kkv = bwd_dkdv_kernel<T, D, MODE, MASK>;
    int rc = allow_lds(reinterpret_cast<const void *>(kq), Cfg::DQ_LDS);
    if (rc == 0) rc = allow_lds(reinterpret_cast<const void *>(kkv), Cfg::DKV_LDS);
    if (rc != 0) return rc;
    hipLaunchKernelGGL(kkv, dim3((unsigned)kv_blocks), dim3(BWD_NT), Cfg::DKV_LDS, stream, p);
    hipLaunchKernelGGL(kq, dim3((unsigned)blocks), dim3(BWD_NT), Cfg::DQ_LDS, stream, p);
    return hipGetLastError() == hipSuccess ? 0 : -6;
  }
}

template <typename T, int D, int MASK>
static int launch_bwd_mask(const BwdParams &p, bool dual, bool tangent_grads, hipStream_t stream) {
  const long long rows = (long long)p.pr.Z * p.pr.H * p.pr.L;
  constexpr int RPB = BWD_NT / (D / 8);
  hipLaunchKernelGGL((bwd_prepass_kernel<T, D>), dim3((unsigned)((rows + RPB - 1) / RPB)), dim3(BWD_NT), 0,
                     stream, p, rows, dual ? 1 : 0);
  if (hipGetLastError() != hipSuccess) return -6;
  if (!dual) return launch_bwd_mode<T, D, BWD_PLAIN, MASK>(p, stream);
  int rc = launch_bwd_mode<T, D, BWD_DUAL, MASK>(p, stream);
  if (rc == 0 && tangent_grads) rc = launch_bwd_mode<T, D, BWD_TANGENT, MASK>(p, stream);
  return rc;
}

int JVPFA_NAME(const BwdParams &p, int mask, bool dual, bool tangent_grads, hipStream_t stream) {
  switch (mask) {
    case MASK_NONE: return launch_bwd_mask<JVPFA_T, JVPFA_D, MASK_NONE>(p, dual, tangent_grads, stream);
    case MASK_BOOL: return launch_bwd_mask<JVPFA_T, JVPFA_D, MASK_BOOL>(p, dual, tangent_grads, stream);
    case MASK_ADD: return launch_bwd_mask<JVPFA_T, JVPFA_D, MASK_ADD>(p, dual, tangent_grads, stream);
  }
  return -3;
}

}  // namespace jvpfa
