// Argument validation shared by the C ABI entry points.
#pragma once
#include <stdint.h>

#include "../../include/jvpfa.h"
#include "params.hpp"

namespace jvpfa {

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

inline int check_problem(const jvpfa_problem &p) {
  if (p.Z < 1 || p.H < 1 || p.L < 1) return JVPFA_E_SHAPE;
  if (p.D != 32 && p.D != 64 && p.D != 128 && p.D != 256) return JVPFA_E_SHAPE;
  if (p.dtype < JVPFA_BF16 || p.dtype > JVPFA_FP32) return JVPFA_E_DTYPE;
  if (p.mask_kind < JVPFA_MASK_NONE || p.mask_kind > JVPFA_MASK_ADD) return JVPFA_E_DTYPE;
  if (!(p.dropout_p >= 0.f && p.dropout_p < 1.f)) return JVPFA_E_SHAPE;
  if (p.mask_kind != JVPFA_MASK_NONE) {
    if (p.causal) return JVPFA_E_CONFLICT;
    if (!p.mask) return JVPFA_E_NULL;
    for (int i = 0; i < 4; ++i)
      if (p.mask_stride[i] < 0) return JVPFA_E_SHAPE;
  }
  return JVPFA_OK;
}

// Lk, Hk as given by the caller (0 = as q); JVPFA_E_SHAPE if they do not fit
inline int check_kv_shape(const jvpfa_problem &p, int32_t Lk, int32_t Hk) {
  if (Lk < 0 || Hk < 0) return JVPFA_E_SHAPE;
  if (Hk > 0 && (Hk > p.H || p.H % Hk != 0)) return JVPFA_E_SHAPE;
  return JVPFA_OK;
}

inline Problem to_problem(const jvpfa_problem &p, const int32_t *key_limit, const int32_t *tiles_q,
                          const int32_t *tiles_k, int32_t Lk = 0, int32_t Hk = 0, const uint32_t *mask_bits = nullptr) {
  Problem r;
  r.Lk = Lk > 0 ? Lk : p.L;
  r.Hk = Hk > 0 ? Hk : p.H;
  const bool masked = p.mask_kind != JVPFA_MASK_NONE;
  // every kernel walks the tile lists when they are there; without them the key limit applies
  const bool lists = masked;
  r.tiles_q = lists ? tiles_q : nullptr;
  r.tiles_k = lists ? tiles_k : nullptr;
  r.bits_k = p.mask_kind == JVPFA_MASK_BOOL ? mask_bits : nullptr;
  r.klimit = (masked && !r.tiles_q && !r.tiles_k) ? key_limit : nullptr;
  r.chunks = 1;
  r.chunk_tiles = 0;
  r.part = nullptr;
  r.drop_thr = 0;
  r.drop_s0 = r.drop_s1 = 0;
  r.drop_rinv = 1.f;
  if (p.dropout_p > 0.f) {
    const double t = (double)p.dropout_p * 4294967296.0;
    r.drop_thr = t < 1.0 ? 1u : (t > 4294967295.0 ? 4294967295u : (uint32_t)t);
    r.drop_s0 = (uint32_t)p.dropout_seed;
    r.drop_s1 = (uint32_t)(p.dropout_seed >> 32);
    r.drop_rinv = 1.f / (1.f - p.dropout_p);
  }
  r.Z = p.Z;
  r.H = p.H;
  r.L = p.L;
  r.causal = p.causal ? 1 : 0;
  r.scale = p.sm_scale;
  r.mask = p.mask_kind == JVPFA_MASK_NONE ? nullptr : p.mask;
  for (int i = 0; i < 4; ++i) r.ms[i] = p.mask_kind == JVPFA_MASK_NONE ? 0 : p.mask_stride[i];
  return r;
}

// 0..11: (dtype, head-dim) slot in the launcher tables.
inline int slot(const jvpfa_problem &p) { return p.dtype * 4 + (p.D == 32 ? 0 : p.D == 64 ? 1 : p.D == 128 ? 2 : 3); }

}  // namespace jvpfa
