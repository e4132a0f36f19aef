// Small grids: when a launch has fewer workgroups than the GPU has compute units (one sequence of a few
// thousand tokens, a handful of heads), the kernels for 16-bit element types with D = 128 and no mask split
// the streamed tiles of every block of owned rows over several workgroups ("chunks").  Each writes fp32
// partial results to a workspace and a merge kernel combines them with the online-softmax merge (every running
// quantity is linear in p once the reference points m and c are made common).  Forward only: the backward of
// such a launch runs its dk/dv and dq workgroups side by side in one launch instead (bwd2_both_kernel).  The
// reference has nothing like it (one program per 32 query rows, jvp_attention.py:2474).
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include <atomic>

#include "common.hpp"
#include "params.hpp"

namespace jvpfa {

struct SplitPlan {
  int chunks, chunk_tiles;
};

// blocks: workgroups of the launch without a split; ntiles_max: streamed tiles of its longest block.
inline SplitPlan split_plan(long long blocks, int ntiles_max, int cus) {
  SplitPlan s = {1, ntiles_max};
  if (cus <= 0 || blocks <= 0 || 2 * blocks > cus) return s;
  // one workgroup per compute unit at most: a workgroup has a fixed cost of about three tiles (its first loads,
  // filling and draining the pipeline), so a second round of short chunks costs more than it saves
  long long want = cus / blocks;
  if (want > 8) want = 8;
  if (want > ntiles_max / 2) want = ntiles_max / 2;    // a chunk is at least two tiles
  if (want < 2) return s;
  s.chunk_tiles = (int)((ntiles_max + want - 1) / want);
  s.chunks = (ntiles_max + s.chunk_tiles - 1) / s.chunk_tiles;
  return s;
}

// Compute units of the current device (0 if it cannot be asked), looked up once per device.  Callable from any
// thread: the cache is atomic, and two threads that both find it empty store the same value.
inline int device_cus() {
  static std::atomic<int> cached[64];
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 0;
  int n = cached[dev].load(std::memory_order_relaxed);
  if (n == 0) {
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) n = 0;
    n = n > 0 ? n : -1;
    cached[dev].store(n, std::memory_order_relaxed);
  }
  return n > 0 ? n : 0;
}

// Workspace of the forward: per chunk and query row 2 D accumulator values (O, T, not yet divided by l) and
// four statistics (m, l, mu_acc, c).
inline size_t fwd_part_floats(int chunks, long long rows, int D) { return (size_t)chunks * rows * (2 * (size_t)D + 4); }
// The kernels that can split: 16-bit element types, D = 128, no mask (the software-pipelined forward and the
// direct-to-LDS backward kernels).  Tiles are 64 wide, blocks 128 rows.
template <typename P> inline bool split_capable(const P &p) {
  return p.dtype != 2 && p.D == 128 && p.mask_kind == 0 && !(p.dropout_p > 0.f);
}
template <typename P> inline SplitPlan fwd_split_plan(const P &p, int Lk) {
  SplitPlan none = {1, 0};
  if (!split_capable(p)) return none;
  const long long blocks = (long long)((p.L + 127) / 128) * p.Z * p.H;
  int keys = Lk;  // of the longest query block (causal: the last one sees keys up to its own last row)
  if (p.causal && ((p.L + 127) / 128) * 128 < keys) keys = ((p.L + 127) / 128) * 128;
  return split_plan(blocks, (keys + 63) / 64, device_cus());
}

// ---- merge kernels -------------------------------------------------------------------------------
// Forward.  part = [chunk][row][2][D] accumulators, then [chunk][row][4] statistics.  One thread per (row, 8
// columns).  With m the largest reference point of the row's chunks and w_c = 2^(m_c - m):
//   l = sum w_c l_c,  O = sum w_c O_c,  and, with c the reference of S' of the heaviest chunk,
//   T = sum w_c (T_c + (c_c - c) O_c),  mu_acc = sum w_c (mu_c + (c_c - c) l_c);
// then the epilogue of the forward kernels: O / l, O' = T / l - (mu_acc / l) O, M = m + log2 l, mu = mu_acc / l + c.
template <typename T, int D, bool DUAL>
__global__ __launch_bounds__(256) void fwd_merge_kernel(const float *part, int chunks, long long rows, T *o, T *ot,
                                                        float *M, float *mu) {
  constexpr int LPR = D / 8;
  const long long row = (long long)blockIdx.x * (256 / LPR) + threadIdx.x / LPR;
  const int d0 = (threadIdx.x % LPR) * 8;
  if (row >= rows) return;
  const float *stat = part + (size_t)chunks * rows * 2 * D;
  float m = -__builtin_inff();
  for (int c = 0; c < chunks; ++c) m = fmaxf(m, stat[((size_t)c * rows + row) * 4]);
  float l = 0.f, best = -1.f, cref = 0.f;
  for (int c = 0; c < chunks; ++c) {
    const float *st = stat + ((size_t)c * rows + row) * 4;
    const float w = (st[0] == -__builtin_inff()) ? 0.f : __builtin_amdgcn_exp2f(st[0] - m);
    l += w * st[1];
    if (w * st[1] > best) {
      best = w * st[1];
      cref = st[3];
    }
  }
  float O[8], Tt[8], mua = 0.f;
#pragma unroll
  for (int e = 0; e < 8; ++e) O[e] = Tt[e] = 0.f;
  for (int c = 0; c < chunks; ++c) {
    const float *st = stat + ((size_t)c * rows + row) * 4;
    const float w = (st[0] == -__builtin_inff()) ? 0.f : __builtin_amdgcn_exp2f(st[0] - m);
    if (w == 0.f) continue;
    const float *acc = part + ((size_t)c * rows + row) * 2 * D + d0;
    const float dc = st[3] - cref;
    mua += w * (st[2] + dc * st[1]);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float oc = acc[e];
      O[e] += w * oc;
      if constexpr (DUAL) Tt[e] += w * (acc[D + e] + dc * oc);
    }
  }
  const bool dead = !(l > 0.f);
  const float inv = dead ? 0.f : 1.f / l, mu_n = mua * inv;
  float o8[8], t8[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    o8[e] = O[e] * inv;
    t8[e] = Tt[e] * inv - mu_n * o8[e];
  }
  store8<T>(o + (size_t)row * D + d0, o8);
  if constexpr (DUAL) store8<T>(ot + (size_t)row * D + d0, t8);
  if (d0 == 0) {
    M[row] = dead ? __builtin_inff() : m + __builtin_amdgcn_logf(l);
    if constexpr (DUAL) mu[row] = dead ? 0.f : mu_n + cref;
  }
}

}  // namespace jvpfa
