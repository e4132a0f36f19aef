// C ABI: jvpfa_mask_tiles -- lists of the 64-wide tiles of a mask that hold an attended entry.
//
// The forward and dq kernels own 128 query rows and stream 64-key tiles; the dk/dv kernels own 128
// keys and stream 64-query tiles.  One workgroup here walks the strip of one such owner and writes
// the indices of the tiles worth visiting, so that the attention kernels skip the rest.  The
// reference has nothing like it: it reads and applies the whole (Z,H,L,L) mask
// (jvp_attention.py:2383-2388, :241-251).
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <algorithm>

#include "api_common.hpp"

namespace jvpfa {

template <typename E, bool BOOL> __device__ __forceinline__ bool attended(E x) {
  if constexpr (BOOL) return x != 0;
  else return (float)x != -__builtin_inff();
}

// KEYS_OWNED false: block = 128 query rows, tiles run over keys (list for forward / dq).
// KEYS_OWNED true:  block = 128 keys, tiles run over query rows (list for dk/dv).
// Every thread looks at 32 consecutive keys of one row of the current tile.
template <typename E, bool BOOL, bool KEYS_OWNED>
__global__ __launch_bounds__(256) void mask_tiles_kernel(const E *mask, int64_t s0, int64_t s1, int64_t s2,
                                                         int64_t s3, int hm, int Lq, int Lk, int *out) {
  // owned: the axis cut into blocks of 128; streamed: the axis cut into tiles of 64
  const int owned = KEYS_OWNED ? Lk : Lq, streamed = KEYS_OWNED ? Lq : Lk;
  const int nblk = (owned + TILE_BLOCK - 1) / TILE_BLOCK, nt = (streamed + TILE_W - 1) / TILE_W;
  const int plane = blockIdx.x / nblk, blk = blockIdx.x % nblk;
  const E *base = mask + (int64_t)(plane / hm) * s0 + (int64_t)(plane % hm) * s1;
  int *list = out + ((size_t)plane * nblk + blk) * (size_t)(nt + 1);
  const int tid = threadIdx.x;
  constexpr int PARTS = KEYS_OWNED ? 4 : 2;  // 32-key pieces per row of a tile
  const int rsub = tid / PARTS, part = tid % PARTS;
  // 16-byte vector reads when every piece starts on a 16-byte boundary
  constexpr int VEC = 16 / sizeof(E);
  const bool vec_ok = s3 == 1 && (s0 % VEC) == 0 && (s1 % VEC) == 0 && (s2 % VEC) == 0 &&
                      (reinterpret_cast<uintptr_t>(mask) % 16) == 0;
  int count = 0;
  constexpr int U = 4;  // tiles looked at per round: their loads are all in flight before the first vote
  for (int t0 = 0; t0 < nt; t0 += U) {
    bool any[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int t = t0 + u;
      const int row = KEYS_OWNED ? t * TILE_W + rsub : blk * TILE_BLOCK + rsub;
      const int key0 = (KEYS_OWNED ? blk * TILE_BLOCK : t * TILE_W) + 32 * part;
      any[u] = false;
      if (t < nt && row < Lq && key0 < Lk) {
        const E *rp = base + (int64_t)row * s2;
        if (vec_ok && key0 + 32 <= Lk) {
#pragma unroll
          for (int v = 0; v < 32 / VEC; ++v) {
            const uint4 w = *reinterpret_cast<const uint4 *>(rp + key0 + v * VEC);
            if constexpr (BOOL) {
              any[u] |= (w.x | w.y | w.z | w.w) != 0;
            } else {
              E e[VEC];
              __builtin_memcpy(e, &w, 16);
#pragma unroll
              for (int i = 0; i < VEC; ++i) any[u] |= attended<E, BOOL>(e[i]);
            }
          }
        } else {
          const int n = min(32, Lk - key0);
          for (int i = 0; i < n; ++i) any[u] |= attended<E, BOOL>(rp[(int64_t)(key0 + i) * s3]);
        }
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (__syncthreads_or(any[u])) {  // uniform over the workgroup
        if (tid == 0) list[1 + count] = t0 + u;
        ++count;
      }
    }
  }
  if (tid == 0) {
    // a strip without any attended entry still visits one (fully masked) tile, which keeps its
    // output rows defined: zeros
    if (count == 0) list[1] = 0;
    list[0] = count == 0 ? 1 : count;
  }
}

template <typename E, bool BOOL>
static int launch_both(const jvpfa_problem &p, int Lk, int *tq, int *tk, hipStream_t stream) {
  const int hm = p.mask_stride[1] ? p.H : 1, zm = p.mask_stride[0] ? p.Z : 1;
  const long long qblocks = (long long)zm * hm * ((p.L + TILE_BLOCK - 1) / TILE_BLOCK);
  const long long kblocks = (long long)zm * hm * ((Lk + TILE_BLOCK - 1) / TILE_BLOCK);
  if (qblocks > 0x7fffffffLL || kblocks > 0x7fffffffLL) return JVPFA_E_SHAPE;
  const E *m = static_cast<const E *>(p.mask);
  const int64_t *s = p.mask_stride;
  if (tq)
    hipLaunchKernelGGL((mask_tiles_kernel<E, BOOL, false>), dim3((unsigned)qblocks), dim3(256), 0, stream, m, s[0],
                       s[1], s[2], s[3], hm, p.L, Lk, tq);
  if (tk)
    hipLaunchKernelGGL((mask_tiles_kernel<E, BOOL, true>), dim3((unsigned)kblocks), dim3(256), 0, stream, m, s[0],
                       s[1], s[2], s[3], hm, p.L, Lk, tk);
  return hipGetLastError() == hipSuccess ? JVPFA_OK : JVPFA_E_LAUNCH;
}

// Boolean mask -> a pair of words per (tile of 64 query rows, key): bit i of word hf = entry (query
// 64 t + 32 hf + i, key) != 0.  A thread owns four consecutive keys of one half tile (32 rows); a workgroup
// 1024 keys.  HBM-bound: reads the mask
// once (four bytes per thread and row, the rows of a block all in flight), writes an eighth of it.
__global__ __launch_bounds__(256) void mask_bits_kernel(const uint8_t *mask, int64_t s0, int64_t s1, int64_t s2,
                                                        int64_t s3, int hm, int Lq, int Lk, int kchunks,
                                                        uint32_t *out) {
  const int nqb = 2 * ((Lq + 63) / 64);  // half tiles, an even number: the last may lie wholly past the last row
  const int kc = blockIdx.x % kchunks;
  const int qb = (blockIdx.x / kchunks) % nqb;
  const int plane = blockIdx.x / kchunks / nqb;
  const int key0 = kc * 1024 + 4 * threadIdx.x;
  if (key0 >= Lk) return;
  const uint8_t *base = mask + (int64_t)(plane / hm) * s0 + (int64_t)(plane % hm) * s1 + (int64_t)key0 * s3;
  const int rows = max(0, min(32, Lq - 32 * qb));
  const bool vec = s3 == 1 && key0 + 4 <= Lk && ((reinterpret_cast<uintptr_t>(base) | (uintptr_t)s2) & 3u) == 0;
  uint32_t w[4] = {0u, 0u, 0u, 0u};
  if (vec) {
    uint32_t x[32];
#pragma unroll
    for (int i = 0; i < 32; ++i)
      x[i] = i < rows ? *reinterpret_cast<const uint32_t *>(base + (int64_t)(32 * qb + i) * s2) : 0u;
#pragma unroll
    for (int i = 0; i < 32; ++i) {
#pragma unroll
      for (int j = 0; j < 4; ++j) w[j] |= ((x[i] >> (8 * j)) & 0xffu) ? (1u << i) : 0u;
    }
  } else {
    const int nk = min(4, Lk - key0);
    for (int i = 0; i < rows; ++i) {
      const uint8_t *rp = base + (int64_t)(32 * qb + i) * s2;
      for (int j = 0; j < nk; ++j) w[j] |= rp[(int64_t)j * s3] ? (1u << i) : 0u;
    }
  }
  // (a plane has ceil(Lq / 64) tiles; the second half of a last tile that ends early is written as zeros by
  // the workgroups of the block of rows that does not exist: see the launch)
  uint32_t *dst = out + (((size_t)plane * (nqb / 2) + qb / 2) * (size_t)Lk + key0) * 2 + (qb & 1);
  for (int j = 0; j < min(4, Lk - key0); ++j) dst[2 * j] = w[j];
}
}  // namespace jvpfa

using namespace jvpfa;

namespace jvpfa {
__global__ __launch_bounds__(256) void dropout_keep_kernel(Problem pr, uint64_t n, uint8_t *keep) {
  // a launch holds fewer than 2^32 threads, the pattern may hold more entries: each thread strides over the rest
  for (uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (uint64_t)gridDim.x * 256) {
    const uint64_t row = i / (uint64_t)pr.Lk;  // (z H + h) L + query
    keep[i] = drop_scale(pr, (int)(row / (uint64_t)pr.L), (int)(row % (uint64_t)pr.L), (int)(i % (uint64_t)pr.Lk)) != 0.f;
  }
}
}  // namespace jvpfa

extern "C" int jvpfa_dropout_keep(const jvpfa_problem *p, int32_t Lk, uint8_t *keep, void *hip_stream) {
  if (!p || !keep) return JVPFA_E_NULL;
  if (p->Z < 1 || p->H < 1 || p->L < 1 || Lk < 0 || !(p->dropout_p >= 0.f && p->dropout_p < 1.f)) return JVPFA_E_SHAPE;
  jvpfa_problem q = *p;
  q.mask_kind = JVPFA_MASK_NONE;
  const Problem pr = to_problem(q, nullptr, nullptr, nullptr, Lk, 0);
  const uint64_t n = (uint64_t)p->Z * p->H * p->L * pr.Lk;  // entry (z, h, i, j) is byte ((z H + h) L + i) Lk + j
  if (n == 0) return JVPFA_OK;
  const uint64_t blocks = std::min<uint64_t>((n + 255) / 256, 1u << 20);
  hipLaunchKernelGGL(dropout_keep_kernel, dim3((unsigned)blocks), dim3(256), 0, static_cast<hipStream_t>(hip_stream), pr, n, keep);
  return hipGetLastError() == hipSuccess ? JVPFA_OK : JVPFA_E_LAUNCH;
}

extern "C" size_t jvpfa_mask_tiles_bytes(const jvpfa_problem *p, int32_t Lk, int32_t keys_owned) {
  if (!p || p->Z < 1 || p->H < 1 || p->L < 1 || Lk < 0) return 0;
  const size_t planes = (size_t)(p->mask_stride[0] ? p->Z : 1) * (p->mask_stride[1] ? p->H : 1);
  const size_t lk = Lk > 0 ? Lk : p->L, owned = keys_owned ? lk : p->L, streamed = keys_owned ? p->L : lk;
  const size_t nblk = (owned + TILE_BLOCK - 1) / TILE_BLOCK, nt = (streamed + TILE_W - 1) / TILE_W;
  return planes * nblk * (nt + 1) * sizeof(int32_t);
}

extern "C" int jvpfa_mask_tiles(const jvpfa_problem *p, int32_t Lk, int32_t *tiles_q, int32_t *tiles_k, void *hip_stream) {
  if (!p || (!tiles_q && !tiles_k)) return JVPFA_E_NULL;
  if (p->Z < 1 || p->H < 1 || p->L < 1 || Lk < 0) return JVPFA_E_SHAPE;
  if (p->dtype < JVPFA_BF16 || p->dtype > JVPFA_FP32) return JVPFA_E_DTYPE;
  if (p->mask_kind != JVPFA_MASK_BOOL && p->mask_kind != JVPFA_MASK_ADD) return JVPFA_E_DTYPE;
  if (!p->mask) return JVPFA_E_NULL;
  for (int i = 0; i < 4; ++i)
    if (p->mask_stride[i] < 0) return JVPFA_E_SHAPE;
  hipStream_t stream = static_cast<hipStream_t>(hip_stream);
  const int lk = Lk > 0 ? Lk : p->L;
  if (p->mask_kind == JVPFA_MASK_BOOL) return launch_both<uint8_t, true>(*p, lk, tiles_q, tiles_k, stream);
  switch (p->dtype) {
    case JVPFA_BF16: return launch_both<__bf16, false>(*p, lk, tiles_q, tiles_k, stream);
    case JVPFA_FP16: return launch_both<_Float16, false>(*p, lk, tiles_q, tiles_k, stream);
    default: return launch_both<float, false>(*p, lk, tiles_q, tiles_k, stream);
  }
}

static inline size_t mask_planes(const jvpfa_problem *p) {
  return (size_t)(p->mask_stride[0] ? p->Z : 1) * (p->mask_stride[1] ? p->H : 1);
}

extern "C" size_t jvpfa_mask_bits_bytes(const jvpfa_problem *p, int32_t Lk) {
  if (!p || p->Z < 1 || p->H < 1 || p->L < 1 || Lk < 0) return 0;
  const size_t lk = Lk > 0 ? Lk : p->L;
  return mask_planes(p) * (((size_t)p->L + 63) / 64) * lk * 2 * sizeof(uint32_t);
}

extern "C" int jvpfa_mask_bits(const jvpfa_problem *p, int32_t Lk, uint32_t *bits, void *hip_stream) {
  if (!p || !bits) return JVPFA_E_NULL;
  if (p->Z < 1 || p->H < 1 || p->L < 1 || Lk < 0) return JVPFA_E_SHAPE;
  if (p->mask_kind != JVPFA_MASK_BOOL) return JVPFA_E_DTYPE;
  if (!p->mask) return JVPFA_E_NULL;
  for (int i = 0; i < 4; ++i)
    if (p->mask_stride[i] < 0) return JVPFA_E_SHAPE;
  if (reinterpret_cast<uintptr_t>(bits) & 7u) return JVPFA_E_ALIGN;
  const int lk = Lk > 0 ? Lk : p->L;
  const int hm = p->mask_stride[1] ? p->H : 1, kchunks = (lk + 1023) / 1024;
  const long long blocks = (long long)mask_planes(p) * (2 * ((p->L + 63) / 64)) * kchunks;
  if (blocks > 0x7fffffffLL) return JVPFA_E_SHAPE;
  const int64_t *s = p->mask_stride;
  hipLaunchKernelGGL(mask_bits_kernel, dim3((unsigned)blocks), dim3(256), 0, static_cast<hipStream_t>(hip_stream),
                     static_cast<const uint8_t *>(p->mask), s[0], s[1], s[2], s[3], hm, p->L, lk, kchunks, bits);
  return hipGetLastError() == hipSuccess ? JVPFA_OK : JVPFA_E_LAUNCH;
}
