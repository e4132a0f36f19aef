// Kernel-side argument blocks (the C ABI structs of include/jvpfa.h, already validated).
#pragma once
#include <stdint.h>

namespace jvpfa {

enum MaskKind { MASK_NONE = 0, MASK_BOOL = 1, MASK_ADD = 2 };

struct Problem {
  int Z, H, L;
  int causal;
  float scale;
  const void *mask;
  int64_t ms[4];  // element strides (z, h, query, key)
  const int *klimit;  // per batch entry: keys at or past this index are masked by the mask (hint), or null
};

struct FwdParams {
  Problem pr;
  const void *q, *k, *v, *qt, *kt, *vt;
  void *o, *ot;
  float *M, *mu;
};

struct BwdParams {
  Problem pr;
  const void *q, *k, *v, *qt, *kt, *vt, *o, *ot;
  const float *M, *mu;
  const void *go, *gt;
  void *dq, *dk, *dv, *dqt, *dkt, *dvt;
  float *d1, *a, *d2;  // row statistics produced by the pre-pass, each (Z, H, L)
};

// What a backward launch computes.
//   BWD_PLAIN    gradient of <gO,O> only (no tangents anywhere): dq / dk,dv
//   BWD_DUAL     gradient of <gO,O> + <gT,O'> w.r.t. the primal inputs: dq / dk,dv
//   BWD_TANGENT  gradient of <gT,O'> w.r.t. the tangent inputs: dqt / dkt,dvt
enum BwdMode { BWD_PLAIN = 0, BWD_DUAL = 1, BWD_TANGENT = 2 };

}  // namespace jvpfa
