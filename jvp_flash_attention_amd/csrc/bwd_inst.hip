// One translation unit per (element type, head dim): compiled with
//   -DJVPFA_T=<__bf16|_Float16|float> -DJVPFA_D=<32|64|128|256> -DJVPFA_NAME=<symbol>
// and exporting  int JVPFA_NAME(const BwdParams&, int mask_kind, bool dual, bool tangent_grads,
// hipStream_t): pre-pass, then the dq and dk/dv kernels of every requested mode.
#include "bwd_kernel.hpp"
#include "bwd_kernel_v2.hpp"
#include "bwd_kernel_wide.hpp"
#include "bwd_kernel_pair.hpp"
#include "launch.hpp"
#include "split.hpp"

namespace jvpfa {

// Which of the tangent-input gradients the dual kernels of the direct-to-LDS family produce on the way when
// all six gradients are asked for (dq' costs the dq kernel one more product per tile and dk', dv' the dk/dv
// kernel two, against a second pair of launches that forms the score tiles again): dq' wherever that family
// runs; dk', dv' where the two extra accumulators fit (D <= 64; at D = 64 that kernel then has a compute unit
// to itself instead of sharing it with a second workgroup and is still 4 - 9 % ahead; at D = 128 dK, dV, the
// resident K, V, K' and the tiles already take 452 of the 512 registers and dK', dV' would add 128).
template <typename T, int D> struct BwdFold {
  static constexpr bool DQ = sizeof(T) == 2;
  static constexpr bool KV = sizeof(T) == 2 && D <= 64;
};

// The dk/dv kernel of the direct-to-LDS family for one launch.  MK is MASK, or MASK_BITS for a boolean mask
// whose bit-packed copy the caller handed over.  fold_kv: the dual variant that also writes dk', dv'.
template <typename T, int D, int MODE, int MK>
static auto pick_dkdv(bool no_go, bool grouped, bool fold_kv, bool drop) -> void (*)(const BwdParams) {
  constexpr bool NG = MODE != BWD_DUAL;  // the GO template argument of the kernels without gO
  if (drop) {
    if (grouped) return no_go ? bwd2_dkdv_kernel<T, D, MODE, MK, NG, true, false, true> : bwd2_dkdv_kernel<T, D, MODE, MK, true, true, false, true>;
    return no_go ? bwd2_dkdv_kernel<T, D, MODE, MK, NG, false, false, true> : bwd2_dkdv_kernel<T, D, MODE, MK, true, false, false, true>;
  }
  if constexpr (MODE == BWD_DUAL && BwdFold<T, D>::KV) {
    if (fold_kv) {
      if (grouped) return no_go ? bwd2_dkdv_kernel<T, D, MODE, MK, false, true, true> : bwd2_dkdv_kernel<T, D, MODE, MK, true, true, true>;
      return no_go ? bwd2_dkdv_kernel<T, D, MODE, MK, false, false, true> : bwd2_dkdv_kernel<T, D, MODE, MK, true, false, true>;
    }
  }
  // D = 64: the register-capped twins, two workgroups per compute unit (D = 32 needs no cap for that); the masked
  // dual kernel needs a few registers more than the cap leaves
  if constexpr (D == 64 && (MK == MASK_NONE || MODE != BWD_DUAL)) {
    if (grouped) return no_go ? bwd2_dkdv_kernel_2wg<T, D, MODE, MK, NG, true> : bwd2_dkdv_kernel_2wg<T, D, MODE, MK, true, true>;
    return no_go ? bwd2_dkdv_kernel_2wg<T, D, MODE, MK, NG> : bwd2_dkdv_kernel_2wg<T, D, MODE, MK, true>;
  }
  if (grouped) return no_go ? bwd2_dkdv_kernel<T, D, MODE, MK, NG, true> : bwd2_dkdv_kernel<T, D, MODE, MK, true, true>;
  return no_go ? bwd2_dkdv_kernel<T, D, MODE, MK, NG> : bwd2_dkdv_kernel<T, D, MODE, MK, true>;
}
// An additive mask can be streamed through LDS as tiles (MASK_TILE) when its rows are runs of contiguous keys
// that start on 16-byte boundaries wherever a tile starts, and 64 rows stay within a 32-bit offset.
template <typename T> static bool mask_rows_tileable(const Problem &pr) {
  const int64_t es = sizeof(T);
  if (pr.ms[3] != 1 || (reinterpret_cast<uintptr_t>(pr.mask) & 15u)) return false;
  for (int i = 0; i < 3; ++i)
    if (pr.ms[i] < 0 || (pr.ms[i] * es) % 16 != 0) return false;
  return 64 * pr.ms[2] * es < ((int64_t)1 << 31);
}
// *lds: the dynamic LDS bytes of the kernel returned
template <typename T, int D, int MODE, int MASK>
static auto pick_dkdv_for(const BwdParams &p, bool no_go, bool grouped, bool fold_kv, bool drop, size_t *lds) -> void (*)(const BwdParams) {
  using Cfg2 = Bwd2Cfg<T, D, MODE>;
  *lds = Cfg2::DKV_LDS;
  if constexpr (MASK == MASK_BOOL) {
    if (p.pr.bits_k) return pick_dkdv<T, D, MODE, MASK_BITS>(no_go, grouped, fold_kv, drop);
  }
  if constexpr (MASK == MASK_ADD) {
    if (mask_rows_tileable<T>(p.pr)) {
      *lds = Cfg2::DKV_LDS_MTILE;
      return pick_dkdv<T, D, MODE, MASK_TILE>(no_go, grouped, fold_kv, drop);
    }
  }
  return pick_dkdv<T, D, MODE, MASK>(no_go, grouped, fold_kv, drop);
}

// six: all six gradients were asked for.  The dual launch then also writes what BwdFold says, and the tangent
// launch skips the kernels whose outputs exist already.
template <typename T, int D, int MODE, int MASK>
static int launch_bwd_mode(const BwdParams &p, bool six, hipStream_t stream) {
  using Cfg = BwdCfg<T, D, MODE>;
  const int nb = (p.pr.L + BWD_BLK - 1) / BWD_BLK;
  const long long blocks = (long long)nb * p.pr.Z * p.pr.H;
  if (blocks > 0x7fffffffLL) return -2;
  // the dk/dv kernels run one workgroup per 128 keys of a key/value head (the same count as for dq
  // when k, v have q's shape)
  const long long kv_blocks = (long long)((p.pr.Lk + BWD_BLK - 1) / BWD_BLK) * p.pr.Z * p.pr.Hk;
  if (kv_blocks > 0x7fffffffLL) return -2;
  if (p.pr.drop_thr != 0) {
    // dropout: the direct-to-LDS kernels carry it for the 16-bit types, the register-staged ones for fp32
    if constexpr (sizeof(T) == 2 && D <= 128) {
      using Cfg2 = Bwd2Cfg<T, D, MODE>;
      const bool no_go = MODE == BWD_DUAL && p.go == nullptr;
      constexpr bool NG = MODE != BWD_DUAL;
      const bool grouped = p.pr.Hk != p.pr.H;
      void (*kq)(const BwdParams) = no_go ? bwd2_dq_kernel<T, D, MODE, MASK, NG, false, true> : bwd2_dq_kernel<T, D, MODE, MASK, true, false, true>;
      size_t kv_lds = 0;
      void (*kkv)(const BwdParams) = pick_dkdv_for<T, D, MODE, MASK>(p, no_go, grouped, false, true, &kv_lds);
      int rc = allow_lds(reinterpret_cast<const void *>(kq), Cfg2::DQ_LDS);
      if (rc == 0) rc = allow_lds(reinterpret_cast<const void *>(kkv), kv_lds);
      if (rc != 0) return rc;
      hipLaunchKernelGGL(kkv, dim3((unsigned)kv_blocks), dim3(Cfg2::NT), kv_lds, stream, p);
      hipLaunchKernelGGL(kq, dim3((unsigned)blocks), dim3(Cfg2::NT), Cfg2::DQ_LDS, stream, p);
      return hipGetLastError() == hipSuccess ? 0 : -6;
    } else if constexpr (sizeof(T) == 2 && D == 256 && MODE == BWD_DUAL) {
      using CfgP = BwdPairCfg<T, D>;
      const bool no_go = p.go == nullptr;
      const long long qblocks = (long long)((p.pr.L + CfgP::BLK - 1) / CfgP::BLK) * p.pr.Z * p.pr.H;
      const long long kblocks = (long long)((p.pr.Lk + CfgP::BLK - 1) / CfgP::BLK) * p.pr.Z * p.pr.Hk;
      if (qblocks > 0x7fffffffLL || kblocks > 0x7fffffffLL) return -2;
      void (*kq)(const BwdParams) = no_go ? bwdp_dq_kernel<T, D, MASK, false, false, true> : bwdp_dq_kernel<T, D, MASK, true, false, true>;
      void (*kkv)(const BwdParams) = no_go ? bwdp_dkdv_kernel<T, D, MASK, false, true> : bwdp_dkdv_kernel<T, D, MASK, true, true>;
      int rc = allow_lds(reinterpret_cast<const void *>(kq), CfgP::DQ_LDS);
      if (rc == 0) rc = allow_lds(reinterpret_cast<const void *>(kkv), CfgP::DKV_LDS);
      if (rc != 0) return rc;
      hipLaunchKernelGGL(kkv, dim3((unsigned)kblocks), dim3(CfgP::NT), CfgP::DKV_LDS, stream, p);
      hipLaunchKernelGGL(kq, dim3((unsigned)qblocks), dim3(CfgP::NT), CfgP::DQ_LDS, stream, p);
      return hipGetLastError() == hipSuccess ? 0 : -6;
    } else if constexpr (sizeof(T) == 2 && D == 256) {
      using CfgW = BwdWideCfg<T, D, MODE>;
      using CfgK = BwdWideKvCfg<T, D, MODE>;
      auto kq = bwdw_dq_kernel<T, D, MODE, MASK, true>;
      auto kkv = bwdw_dkdv_kernel<T, D, MODE, MASK, true>;
      int rc = allow_lds(reinterpret_cast<const void *>(kq), CfgW::DQ_LDS);
      if (rc == 0) rc = allow_lds(reinterpret_cast<const void *>(kkv), CfgK::DKV_LDS);
      if (rc != 0) return rc;
      hipLaunchKernelGGL(kkv, dim3((unsigned)kv_blocks), dim3(CfgK::NT), CfgK::DKV_LDS, stream, p);
      hipLaunchKernelGGL(kq, dim3((unsigned)blocks), dim3(CfgW::NT), CfgW::DQ_LDS, stream, p);
      return hipGetLastError() == hipSuccess ? 0 : -6;
    } else {
      auto kq = bwd_dq_kernel<T, D, MODE, MASK, true>;
      auto kkv = bwd_dkdv_kernel<T, D, MODE, MASK, true>;
      int rc = allow_lds(reinterpret_cast<const void *>(kq), Cfg::DQ_LDS);
      if (rc == 0) rc = allow_lds(reinterpret_cast<const void *>(kkv), Cfg::DKV_LDS);
      if (rc != 0) return rc;
      hipLaunchKernelGGL(kkv, dim3((unsigned)kv_blocks), dim3(BWD_NT), Cfg::DKV_LDS, stream, p);
      hipLaunchKernelGGL(kq, dim3((unsigned)blocks), dim3(BWD_NT), Cfg::DQ_LDS, stream, p);
      return hipGetLastError() == hipSuccess ? 0 : -6;
    }
  }
  if constexpr (sizeof(T) == 2 && D <= 128) {  // direct-to-LDS, double-buffered kernels
   {
    using Cfg2 = Bwd2Cfg<T, D, MODE>;
    // gO may be absent only in the dual mode (loss depends on O' alone)
    const bool no_go = MODE == BWD_DUAL && p.go == nullptr;
    constexpr bool NG = MODE != BWD_DUAL;  // the GO template argument of the kernels without gO
    void (*kq)(const BwdParams), (*kkv)(const BwdParams);
    const bool grouped = p.pr.Hk != p.pr.H;  // a key/value head serves several query heads
    using Fold = BwdFold<T, D>;
    bool run_q = true, run_kv = true;
    if constexpr (MODE == BWD_TANGENT) {
      run_q = !(six && Fold::DQ);
      run_kv = !(six && Fold::KV);
    }
    if constexpr (MODE == BWD_DUAL) {
      if (six) {  // the variants that also write dq' (and dk', dv')
        // (without gO the register cap of the two-workgroup twin makes the allocator copy LDS fragments out of
        // their registers before they have arrived, which the build's lint refuses: that variant runs uncapped)
        if constexpr (D == 64) kq = no_go ? bwd2_dq_kernel<T, D, MODE, MASK, false, true> : bwd2_dq_kernel_2wg<T, D, MODE, MASK, true, true>;
        else kq = no_go ? bwd2_dq_kernel<T, D, MODE, MASK, false, true> : bwd2_dq_kernel<T, D, MODE, MASK, true, true>;
      }
    }
    const bool plain_q = !(MODE == BWD_DUAL && six);
    if constexpr (D == 64) {  // the register-capped twins: two workgroups per compute unit (D = 32 needs no cap for that)
      if (plain_q) kq = no_go ? bwd2_dq_kernel_2wg<T, D, MODE, MASK, NG> : bwd2_dq_kernel_2wg<T, D, MODE, MASK, true>;
    } else {
      if (plain_q) kq = no_go ? bwd2_dq_kernel<T, D, MODE, MASK, NG> : bwd2_dq_kernel<T, D, MODE, MASK, true>;
      if constexpr (D == 128 && MODE == BWD_PLAIN) kq = bwd2_dq_kernel_2wg_plain<T, D, MODE, MASK>;
    }
    size_t kv_lds = 0;
    kkv = pick_dkdv_for<T, D, MODE, MASK>(p, no_go, grouped, MODE == BWD_DUAL && six, false, &kv_lds);
    // a grid smaller than the GPU: both roles in one launch, side by side
    const int cus = device_cus();
    if (!grouped && !six && blocks < cus && kv_blocks < cus) {
      void (*kb)(const BwdParams, int) = no_go ? bwd2_both_kernel<T, D, MODE, MASK, NG> : bwd2_both_kernel<T, D, MODE, MASK, true>;
      constexpr size_t LDS = Cfg2::DKV_LDS > Cfg2::DQ_LDS ? Cfg2::DKV_LDS : Cfg2::DQ_LDS;
      const int rcb = allow_lds(reinterpret_cast<const void *>(kb), LDS);
      if (rcb != 0) return rcb;
      hipLaunchKernelGGL(kb, dim3((unsigned)(kv_blocks + blocks)), dim3(Cfg2::NT), LDS, stream, p, (int)kv_blocks);
      return hipGetLastError() == hipSuccess ? 0 : -6;
    }
    int rc = allow_lds(reinterpret_cast<const void *>(kq), Cfg2::DQ_LDS);
    if (rc == 0) rc = allow_lds(reinterpret_cast<const void *>(kkv), kv_lds);
    if (rc != 0) return rc;
    if (run_kv) hipLaunchKernelGGL(kkv, dim3((unsigned)kv_blocks), dim3(Cfg2::NT), kv_lds, stream, p);
    if (run_q) hipLaunchKernelGGL(kq, dim3((unsigned)blocks), dim3(Cfg2::NT), Cfg2::DQ_LDS, stream, p);
    return hipGetLastError() == hipSuccess ? 0 : -6;
   }
  } else if constexpr (sizeof(T) == 2 && D == 256 && MODE == BWD_DUAL) {
    // pairs of waves that share 32 rows and split the resident operands: every product formed once
    using CfgP = BwdPairCfg<T, D>;
    const bool no_go = p.go == nullptr;
    const long long qblocks = (long long)((p.pr.L + CfgP::BLK - 1) / CfgP::BLK) * p.pr.Z * p.pr.H;
    const long long kblocks = (long long)((p.pr.Lk + CfgP::BLK - 1) / CfgP::BLK) * p.pr.Z * p.pr.Hk;
    if (qblocks > 0x7fffffffLL || kblocks > 0x7fffffffLL) return -2;
    void (*kq)(const BwdParams) = no_go ? bwdp_dq_kernel<T, D, MASK, false> : bwdp_dq_kernel<T, D, MASK, true>;
    if (six) kq = no_go ? bwdp_dq_kernel<T, D, MASK, false, true> : bwdp_dq_kernel<T, D, MASK, true, true>;
    void (*kkv)(const BwdParams) = no_go ? bwdp_dkdv_kernel<T, D, MASK, false> : bwdp_dkdv_kernel<T, D, MASK, true>;
    int rc = allow_lds(reinterpret_cast<const void *>(kq), CfgP::DQ_LDS);
    if (rc == 0) rc = allow_lds(reinterpret_cast<const void *>(kkv), CfgP::DKV_LDS);
    if (rc != 0) return rc;
    hipLaunchKernelGGL(kkv, dim3((unsigned)kblocks), dim3(CfgP::NT), CfgP::DKV_LDS, stream, p);
    hipLaunchKernelGGL(kq, dim3((unsigned)qblocks), dim3(CfgP::NT), CfgP::DQ_LDS, stream, p);
    return hipGetLastError() == hipSuccess ? 0 : -6;
  } else if constexpr (sizeof(T) == 2 && D == 256) {
    // without tangents in the launch two operands stay resident and one workgroup holds all 256 columns
    using CfgW = BwdWideCfg<T, D, MODE>;
    using CfgK = BwdWideKvCfg<T, D, MODE>;
    auto kq = bwdw_dq_kernel<T, D, MODE, MASK>;
    auto kkv = bwdw_dkdv_kernel<T, D, MODE, MASK>;
    int rc = allow_lds(reinterpret_cast<const void *>(kq), CfgW::DQ_LDS);
    if (rc == 0) rc = allow_lds(reinterpret_cast<const void *>(kkv), CfgK::DKV_LDS);
    if (rc != 0) return rc;
    hipLaunchKernelGGL(kkv, dim3((unsigned)kv_blocks), dim3(CfgK::NT), CfgK::DKV_LDS, stream, p);
    // (six: the tangent launch of a six-gradient call, whose dq' the dual launch has written already)
    if (!(MODE == BWD_TANGENT && six)) hipLaunchKernelGGL(kq, dim3((unsigned)blocks), dim3(CfgW::NT), CfgW::DQ_LDS, stream, p);
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
  if (!dual) return launch_bwd_mode<T, D, BWD_PLAIN, MASK>(p, false, stream);
  int rc = launch_bwd_mode<T, D, BWD_DUAL, MASK>(p, tangent_grads, stream);
  if (rc == 0 && tangent_grads) rc = launch_bwd_mode<T, D, BWD_TANGENT, MASK>(p, true, stream);
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
