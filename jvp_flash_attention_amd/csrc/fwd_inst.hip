// One translation unit per (element type, head dim): compiled with
//   -DJVPFA_T=<__bf16|_Float16|float> -DJVPFA_D=<32|64|128|256> -DJVPFA_NAME=<symbol>
// and exporting  int JVPFA_NAME(const FwdParams&, bool dual, int mask_kind, hipStream_t).
#include "fwd_kernel.hpp"
#include "fwd_kernel_v2.hpp"
#include "fwd_kernel_v3.hpp"
#include "fwd_kernel_wide.hpp"
#include "launch.hpp"
#include "split.hpp"

namespace jvpfa {

template <typename T, int D, int BN, bool DUAL, int MASK, bool DROP = false>
static int launch_fwd_one(const FwdParams &p, hipStream_t stream) {
  using Cfg = FwdCfg<T, D, BN, DUAL>;
  auto kern = fwd_kernel<T, D, BN, DUAL, MASK, DROP>;
  int rc = allow_lds(reinterpret_cast<const void *>(kern), Cfg::LDS_BYTES);
  if (rc != 0) return rc;
  const int nqb = (p.pr.L + Cfg::BM - 1) / Cfg::BM;
  const long long blocks = (long long)nqb * p.pr.Z * p.pr.H;
  if (blocks > 0x7fffffffLL) return -2;
  hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(Cfg::NT), Cfg::LDS_BYTES, stream, p);
  return hipGetLastError() == hipSuccess ? 0 : -6;
}

// 16-bit element types with D = 64 or 128 take the direct-to-LDS, double-buffered kernel.
template <typename T, int D, bool DUAL, int MASK, bool DROP = false>
static int launch_fwd2_one(const FwdParams &p, hipStream_t stream) {
  using Cfg = Fwd2Cfg<T, D, DUAL>;
  auto kern = fwd2_kernel<T, D, DUAL, MASK, DROP>;
  int rc = allow_lds(reinterpret_cast<const void *>(kern), Cfg::LDS_BYTES);
  if (rc != 0) return rc;
  const int nqb = (p.pr.L + Cfg::BM - 1) / Cfg::BM;
  const long long blocks = (long long)nqb * p.pr.Z * p.pr.H;
  if (blocks > 0x7fffffffLL) return -2;
  hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(Cfg::NT), Cfg::LDS_BYTES, stream, p);
  return hipGetLastError() == hipSuccess ? 0 : -6;
}

// ... and its software-pipelined form (D = 128).
template <typename T, int D, bool DUAL, int MASK = MASK_NONE, bool DROP = false>
static int launch_fwd3_one(const FwdParams &p, hipStream_t stream) {
  using Cfg = Fwd2Cfg<T, D, DUAL>;
  auto kern = fwd3_kernel<T, D, DUAL, MASK, DROP>;
  int rc = allow_lds(reinterpret_cast<const void *>(kern), Cfg::LDS_BYTES);
  if (rc != 0) return rc;
  const int nqb = (p.pr.L + Cfg::BM - 1) / Cfg::BM;
  const long long blocks = (long long)nqb * p.pr.Z * p.pr.H * p.pr.chunks;
  if (blocks > 0x7fffffffLL) return -2;
  hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(Cfg::NT), Cfg::LDS_BYTES, stream, p);
  if (p.pr.chunks > 1) {  // the chunks' partial results become o, ot, M, mu
    const long long rows = (long long)p.pr.Z * p.pr.H * p.pr.L;
    constexpr int RPB = 256 / (D / 8);
    hipLaunchKernelGGL((fwd_merge_kernel<T, D, DUAL>), dim3((unsigned)((rows + RPB - 1) / RPB)), dim3(256), 0, stream,
                       p.pr.part, p.pr.chunks, rows, reinterpret_cast<T *>(p.o), reinterpret_cast<T *>(p.ot), p.M, p.mu);
  }
  return hipGetLastError() == hipSuccess ? 0 : -6;
}

// D = 256.
template <typename T, int D, bool DUAL, int MASK, bool DROP = false>
static int launch_fwd_wide_one(const FwdParams &p, hipStream_t stream) {
  // Without tangents one workgroup holds all columns.  The dual forward runs that kernel first (O, M)
  // and then the tangent pass (O', mu) with the final M: seven products, where two workgroups with a
  // column half each would compute nine.
  using Cfg = FwdWideCfg<T, D, false>;
  const int nqb = (p.pr.L + Cfg::BM - 1) / Cfg::BM;
  const long long blocks = (long long)nqb * p.pr.Z * p.pr.H;
  if (blocks > 0x7fffffffLL) return -2;
  int rc = 0;
  if constexpr (MASK == MASK_NONE && !DROP && !DUAL) {
    // O and M from the software-pipelined kernel: without tangents its resident Q and accumulator fit at
    // D = 256 too (64-key tiles, two stages of K and V = 128 KB of LDS).  (As the first pass of the dual forward
    // it is 7 % faster as well, but the tangent pass's O' then misses the 2e-2 bar on dq in one test with very
    // peaked rows, where its reference c for S', the first tile's mean, is far from the row's mu.)
    using Cfg3 = Fwd2Cfg<T, D, false>;
    auto k3 = fwd3_kernel<T, D, false>;
    rc = allow_lds(reinterpret_cast<const void *>(k3), Cfg3::LDS_BYTES);
    if (rc != 0) return rc;
    hipLaunchKernelGGL(k3, dim3((unsigned)blocks), dim3(Cfg3::NT), Cfg3::LDS_BYTES, stream, p);
  } else {
    auto kern = fwd_wide_kernel<T, D, false, MASK, false, DROP>;
    rc = allow_lds(reinterpret_cast<const void *>(kern), Cfg::LDS_BYTES);
    if (rc != 0) return rc;
    hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(Cfg::NT), Cfg::LDS_BYTES, stream, p);
  }
  if constexpr (DUAL) {
    using CfgT = FwdWideCfg<T, D, true>;
    auto kt = fwd_wide_kernel<T, D, true, MASK, true, DROP>;
    rc = allow_lds(reinterpret_cast<const void *>(kt), CfgT::LDS_BYTES);
    if (rc != 0) return rc;
    hipLaunchKernelGGL(kt, dim3((unsigned)blocks), dim3(CfgT::NT), CfgT::LDS_BYTES, stream, p);
  }
  return hipGetLastError() == hipSuccess ? 0 : -6;
}

template <typename T, int D, int BN, bool DUAL>
static int launch_fwd_mask(const FwdParams &p, int mask, hipStream_t stream) {
  if (p.pr.drop_thr != 0) {
    // dropout: the direct-to-LDS kernels carry it for the 16-bit types, the register-staged one for fp32
    if constexpr (sizeof(T) == 2 && D == 256) {
      switch (mask) {
        case MASK_NONE: return launch_fwd_wide_one<T, D, DUAL, MASK_NONE, true>(p, stream);
        case MASK_BOOL: return launch_fwd_wide_one<T, D, DUAL, MASK_BOOL, true>(p, stream);
        case MASK_ADD: return launch_fwd_wide_one<T, D, DUAL, MASK_ADD, true>(p, stream);
      }
    } else if constexpr (sizeof(T) == 2 && D <= 128) {
      switch (mask) {
        case MASK_NONE:
          // (with a mask and dropout together the pipelined kernel runs out of registers)
          if constexpr (D == 128) return launch_fwd3_one<T, D, DUAL, MASK_NONE, true>(p, stream);
          else return launch_fwd2_one<T, D, DUAL, MASK_NONE, true>(p, stream);
        case MASK_BOOL: return launch_fwd2_one<T, D, DUAL, MASK_BOOL, true>(p, stream);
        case MASK_ADD: return launch_fwd2_one<T, D, DUAL, MASK_ADD, true>(p, stream);
      }
    } else {
      constexpr int BNG = (sizeof(T) == 4 || D > 128) ? 32 : 64;
      switch (mask) {
        case MASK_NONE: return launch_fwd_one<T, D, BNG, DUAL, MASK_NONE, true>(p, stream);
        case MASK_BOOL: return launch_fwd_one<T, D, BNG, DUAL, MASK_BOOL, true>(p, stream);
        case MASK_ADD: return launch_fwd_one<T, D, BNG, DUAL, MASK_ADD, true>(p, stream);
      }
    }
    return -3;
  }
  if constexpr (sizeof(T) == 2 && D == 256) {
    switch (mask) {
      case MASK_NONE: return launch_fwd_wide_one<T, D, DUAL, MASK_NONE>(p, stream);
      case MASK_BOOL: return launch_fwd_wide_one<T, D, DUAL, MASK_BOOL>(p, stream);
      case MASK_ADD: return launch_fwd_wide_one<T, D, DUAL, MASK_ADD>(p, stream);
    }
    return -3;
  } else if constexpr (sizeof(T) == 2 && D == 128) {
    // the pipelined kernel pays off where a slot has enough matrix work to hide the softmax behind
    switch (mask) {
      case MASK_NONE: return launch_fwd3_one<T, D, DUAL>(p, stream);
      case MASK_BOOL: return launch_fwd3_one<T, D, DUAL, MASK_BOOL>(p, stream);
      case MASK_ADD: return launch_fwd3_one<T, D, DUAL, MASK_ADD>(p, stream);
    }
    return -3;
  } else if constexpr (sizeof(T) == 2 && D < 128) {
    switch (mask) {
      case MASK_NONE: return launch_fwd2_one<T, D, DUAL, MASK_NONE>(p, stream);
      case MASK_BOOL: return launch_fwd2_one<T, D, DUAL, MASK_BOOL>(p, stream);
      case MASK_ADD: return launch_fwd2_one<T, D, DUAL, MASK_ADD>(p, stream);
    }
    return -3;
  } else {
    switch (mask) {
      case MASK_NONE: return launch_fwd_one<T, D, BN, DUAL, MASK_NONE>(p, stream);
      case MASK_BOOL: return launch_fwd_one<T, D, BN, DUAL, MASK_BOOL>(p, stream);
      case MASK_ADD: return launch_fwd_one<T, D, BN, DUAL, MASK_ADD>(p, stream);
    }
    return -3;
  }
}

int JVPFA_NAME(const FwdParams &p, bool dual, int mask, hipStream_t stream) {
  constexpr int BN = (sizeof(JVPFA_T) == 4 || JVPFA_D > 128) ? 32 : 64;  // keys per tile of the LDS-copy kernel
  return dual ? launch_fwd_mask<JVPFA_T, JVPFA_D, BN, true>(p, mask, stream)
              : launch_fwd_mask<JVPFA_T, JVPFA_D, BN, false>(p, mask, stream);
}

}  // namespace jvpfa
