// Mask access shared by forward and backward: eight consecutive keys of one query row.
#pragma once
#include "common.hpp"
#include "params.hpp"

namespace jvpfa {

// Boolean mask bytes (nonzero = attend) for keys key0 .. key0+7 of one query row.
// Keys >= Lk read as "masked".
__device__ __forceinline__ void mask_keep8(const Problem &pr, int64_t rowoff, int key0, bool keep[8]) {
  const uint8_t *base = reinterpret_cast<const uint8_t *>(pr.mask) + rowoff;
  if (pr.ms[3] == 1 && key0 + 8 <= pr.Lk && ((reinterpret_cast<uintptr_t>(base + key0) & 7) == 0)) {
    uint64_t w = *reinterpret_cast<const uint64_t *>(base + key0);
#pragma unroll
    for (int e = 0; e < 8; ++e) keep[e] = ((e < 4 ? (uint32_t)w : (uint32_t)(w >> 32)) & (0xffu << (8 * (e & 3)))) != 0;
  } else {
#pragma unroll
    for (int e = 0; e < 8; ++e) keep[e] = (key0 + e < pr.Lk) ? base[(int64_t)(key0 + e) * pr.ms[3]] != 0 : false;
  }
}

// Additive mask values (element type T) for keys key0 .. key0+7, already multiplied by log2(e).
template <typename T>
__device__ __forceinline__ void mask_bias8(const Problem &pr, int64_t rowoff, int key0, float bias[8]) {
  const T *base = reinterpret_cast<const T *>(pr.mask) + rowoff;
  if (pr.ms[3] == 1 && key0 + 8 <= pr.Lk && ((reinterpret_cast<uintptr_t>(base + key0) & 15) == 0)) {
    Frag<T> w = ld8<T>(base + key0);
#pragma unroll
    for (int e = 0; e < 8; ++e) bias[e] = (float)w[e] * LOG2E;
  } else {
#pragma unroll
    for (int e = 0; e < 8; ++e)
      bias[e] = (key0 + e < pr.Lk) ? (float)base[(int64_t)(key0 + e) * pr.ms[3]] * LOG2E : 0.f;
  }
}

// ---- mask data fetched ahead of its use -----------------------------------------------------------
// The loads above sit right where their values are needed, so their latency is exposed.  When the
// key stride is 1 and every row start is aligned, the eight keys of a lane are one vector load that
// can be issued a whole phase of matrix instructions earlier and decoded later.
template <typename T, int MASK> struct MaskAhead {
  uint64_t w;   // MASK_BOOL: eight bytes
  Frag<T> f;    // MASK_ADD: eight elements
};
template <typename T, int MASK> __device__ __forceinline__ bool mask_rows_aligned(const Problem &pr) {
  constexpr int64_t AL = MASK == MASK_BOOL ? 8 : (int64_t)(16 / sizeof(T));  // in elements
  const uintptr_t base = reinterpret_cast<uintptr_t>(pr.mask);
  return pr.ms[3] == 1 && (pr.ms[0] % AL) == 0 && (pr.ms[1] % AL) == 0 && (pr.ms[2] % AL) == 0 &&
         (base % (MASK == MASK_BOOL ? 8 : 16)) == 0;
}
// keys key0 .. key0+7 must exist (key0 + 8 <= L) and key0 must be a multiple of 8
template <typename T, int MASK>
__device__ __forceinline__ MaskAhead<T, MASK> mask_fetch8(const Problem &pr, int64_t rowoff, int key0) {
  MaskAhead<T, MASK> m;
  if constexpr (MASK == MASK_BOOL) m.w = *reinterpret_cast<const uint64_t *>(reinterpret_cast<const uint8_t *>(pr.mask) + rowoff + key0);
  else m.f = ld8<T>(reinterpret_cast<const T *>(pr.mask) + rowoff + key0);
  return m;
}
// The same for any strides and alignment: eight element loads, packed into the same form.  Keys past
// the end are read from the last key instead (callers mask them by index).
template <typename T, int MASK>
__device__ __forceinline__ MaskAhead<T, MASK> mask_fetch8_any(const Problem &pr, int64_t rowoff, int key0) {
  MaskAhead<T, MASK> m;
  if constexpr (MASK == MASK_BOOL) {
    const uint8_t *base = reinterpret_cast<const uint8_t *>(pr.mask) + rowoff;
    uint32_t lo = 0, hi = 0;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const uint32_t b = base[(int64_t)min(key0 + e, pr.Lk - 1) * pr.ms[3]] != 0 ? 0xffu : 0u;
      if (e < 4) lo |= b << (8 * e);
      else hi |= b << (8 * (e - 4));
    }
    m.w = (uint64_t)lo | ((uint64_t)hi << 32);
  } else {
    const T *base = reinterpret_cast<const T *>(pr.mask) + rowoff;
#pragma unroll
    for (int e = 0; e < 8; ++e) m.f[e] = base[(int64_t)min(key0 + e, pr.Lk - 1) * pr.ms[3]];
  }
  return m;
}
// The same with keys past the end delivered as masked (byte 0 / minus infinity), for callers that apply no limit
// of their own.
template <typename T, int MASK>
__device__ __forceinline__ MaskAhead<T, MASK> mask_fetch8_lim(const Problem &pr, int64_t rowoff, int key0) {
  MaskAhead<T, MASK> m;
  if constexpr (MASK == MASK_BOOL) {
    const uint8_t *base = reinterpret_cast<const uint8_t *>(pr.mask) + rowoff;
    uint32_t lo = 0, hi = 0;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const uint32_t raw = base[(int64_t)min(key0 + e, pr.Lk - 1) * pr.ms[3]];
      const uint32_t b = (raw != 0 && key0 + e < pr.Lk) ? 0xffu : 0u;
      if (e < 4) lo |= b << (8 * e);
      else hi |= b << (8 * (e - 4));
    }
    m.w = (uint64_t)lo | ((uint64_t)hi << 32);
  } else {
    const T *base = reinterpret_cast<const T *>(pr.mask) + rowoff;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const T raw = base[(int64_t)min(key0 + e, pr.Lk - 1) * pr.ms[3]];
      m.f[e] = key0 + e < pr.Lk ? raw : (T)(-__builtin_inff());
    }
  }
  return m;
}
template <typename T, int MASK> __device__ __forceinline__ bool mask_keep_of(const MaskAhead<T, MASK> &m, int e) {
  const uint32_t half = e < 4 ? (uint32_t)m.w : (uint32_t)(m.w >> 32);  // 32-bit tests: 64-bit shifts are slow
  return (half & (0xffu << (8 * (e & 3)))) != 0;
}
// 0 for an attended key, minus infinity for a masked one, from byte K of a word of four mask bytes (two
// instructions: the comparison selects its byte itself).  zero and ninf are vector registers that hold 0 and the
// bits of minus infinity (a literal next to vcc would be one constant-bus operand too many).
template <int K> __device__ __forceinline__ float mask_term_of_byte(uint32_t word, uint32_t zero, uint32_t ninf) {
  float t;
  if constexpr (K == 0) asm("v_cmp_eq_u32_sdwa vcc, %1, %2 src0_sel:BYTE_0 src1_sel:DWORD\n\tv_cndmask_b32_e32 %0, 0, %3, vcc" : "=v"(t) : "v"(word), "v"(zero), "v"(ninf) : "vcc");
  if constexpr (K == 1) asm("v_cmp_eq_u32_sdwa vcc, %1, %2 src0_sel:BYTE_1 src1_sel:DWORD\n\tv_cndmask_b32_e32 %0, 0, %3, vcc" : "=v"(t) : "v"(word), "v"(zero), "v"(ninf) : "vcc");
  if constexpr (K == 2) asm("v_cmp_eq_u32_sdwa vcc, %1, %2 src0_sel:BYTE_2 src1_sel:DWORD\n\tv_cndmask_b32_e32 %0, 0, %3, vcc" : "=v"(t) : "v"(word), "v"(zero), "v"(ninf) : "vcc");
  if constexpr (K == 3) asm("v_cmp_eq_u32_sdwa vcc, %1, %2 src0_sel:BYTE_3 src1_sel:DWORD\n\tv_cndmask_b32_e32 %0, 0, %3, vcc" : "=v"(t) : "v"(word), "v"(zero), "v"(ninf) : "vcc");
  return t;
}
template <typename T, int MASK> __device__ __forceinline__ float mask_bias_of(const MaskAhead<T, MASK> &m, int e) {
  return (float)m.f[e] * LOG2E;
}

// The streamed tiles (W = 32 or 64 rows) that a kernel outside the direct-to-LDS family visits: all of them from
// `start` up to `end`, or those of a caller's list of 64-wide tiles (jvpfa_mask_tiles), each walked as 64 / W
// pieces.  `len` is the length of the streamed axis: it bounds whatever a list holds, and a second piece that
// would start past it is left out.
template <int W> struct TileWalk {
  static_assert(W == 32 || W == 64);
  static constexpr int SUB = TILE_W / W;
  const int *list = nullptr;
  int n = 0, start = 0, tmax = 0;
  __device__ __forceinline__ void init(const int *l, int start_, int end, int len) {
    list = l;
    start = start_;
    tmax = (len + TILE_W - 1) / TILE_W - 1;
    if (!l) {
      n = end > start_ ? (end - start_ + W - 1) / W : 0;
      return;
    }
    const int cnt = min(max(l[0], 1), tmax + 1);
    const int last = min(max(l[cnt], 0), tmax);
    n = SUB * cnt - ((SUB == 2 && last * TILE_W + W >= len) ? 1 : 0);
  }
  __device__ __forceinline__ int at(int it) const {
    if (!list) return start + it * W;
    return min(max(list[1 + it / SUB], 0), tmax) * TILE_W + (it % SUB) * W;
  }
};

}  // namespace jvpfa
