// Backward kernels for  Loss = <gO, O> + <gT, O'>  with P recomputed from the saved
// log-sum-exp M (and mu for the tangent path).
//
//   prepass   d1 = rowsum(gO*O), a = rowsum(gT*O), d2 = d1 + rowsum(gT*O') - a*mu
//   dq        one workgroup per 128 query rows, loop over key tiles
//   dkdv      one workgroup per 128 key rows, loop over query tiles
//
// Replaces the reference's _attn_bwd_preprocess (jvp_attention.py:1384-1411), _attn_bwd_dq
// (:1567-1707) and _attn_bwd_dkdv (:1415-1563), which handle gO only; the gT terms follow
//   dS' = P*(A - a),  dS = P*(gO V^T - d1 + B + A*(S' - mu) - a*S' - d2),  P' = P*(S' - mu)
//   A = gT V^T,  B = gT V'^T
//   dQ = s(dS K + dS' K'), dK = s(dS^T Q + dS'^T Q'), dV = P^T gO + P'^T gT
//   dQ' = s dS' K,         dK' = s dS'^T Q,           dV' = P^T gT          (s = sm_scale)
// Unlike the reference (:1519-1522, :1669-1671) an additive mask is part of the recomputed
// logits.
#pragma once
#include "common.hpp"
#include "mask.hpp"
#include "params.hpp"

namespace jvpfa {

constexpr int BWD_NT = 256;
constexpr int BWD_BLK = 128;  // rows owned by a workgroup (32 per wave)
constexpr int BWD_T = 32;     // rows of the streamed tile

template <typename T, int D>
__global__ __launch_bounds__(256) void bwd_prepass_kernel(const BwdParams p, long long rows, int dual) {
  constexpr int LPR = D / 8;  // lanes per row, 8 elements each
  const long long row = (long long)blockIdx.x * (BWD_NT / LPR) + threadIdx.x / LPR;
  const int part = threadIdx.x % LPR;
  float s1 = 0.f, sa = 0.f, s2 = 0.f;
  if (row < rows) {
    const size_t off = (size_t)row * D + part * 8;
    Frag<T> o = ld8<T>(reinterpret_cast<const T *>(p.o) + off);
    if (p.go) {
      Frag<T> go = ld8<T>(reinterpret_cast<const T *>(p.go) + off);
#pragma unroll
      for (int e = 0; e < 8; ++e) s1 += (float)go[e] * (float)o[e];
    }
    if (dual) {
      Frag<T> gt = ld8<T>(reinterpret_cast<const T *>(p.gt) + off);
      Frag<T> ot = ld8<T>(reinterpret_cast<const T *>(p.ot) + off);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        sa += (float)gt[e] * (float)o[e];
        s2 += (float)gt[e] * (float)ot[e];
      }
    }
  }
#pragma unroll
  for (int w = LPR / 2; w >= 1; w /= 2) {
    s1 += __shfl_xor(s1, w, 64);
    sa += __shfl_xor(sa, w, 64);
    s2 += __shfl_xor(s2, w, 64);
  }
  if (row < rows && part == 0) {
    p.d1[row] = s1;
    if (dual) {
      p.a[row] = sa;
      p.d2[row] = s1 + s2 - sa * p.mu[row];  // BWD_DUAL uses d1 + d2 only, kept in one statistic
    }
  }
}

template <typename T, int D, int MODE> struct BwdCfg {
  static constexpr int PAD = 16 / sizeof(T);
  static constexpr int LDN = D + PAD;       // row-major streamed tiles (32 x D)
  static constexpr int LDT = BWD_T + PAD;   // transposed streamed tiles (D x 32)
  static constexpr int N_ELEMS = BWD_T * LDN;
  static constexpr int T_ELEMS = D * LDT;
  // dq:   PLAIN K,V,K^T | DUAL K,K',V,V',K^T,K'^T | TANGENT K,V,K^T
  // dkdv: PLAIN Q,gO,Q^T,gO^T | DUAL Q,Q',gO,gT + 4 transposed | TANGENT Q,gT,Q^T,gT^T
  // D = 256 (fp32: rows of 1024 bytes; 16-bit types come here with dropout only): a wave's own rows of four
  // operands would be the whole register file (fp32: 4 x 128 registers, next to 128 - 256 of accumulators) and
  // eight 32-row fp32 tiles twice the LDS, so there the own rows are read from global
  // memory where they are used (the same 32 bytes per lane every tile: cache hits) and only the tiles whose
  // fragments run along the streamed index are staged (dq: K, K' both ways; dk/dv: the four transposed ones);
  // the other row-wise fragments also come straight from global memory.
  static constexpr bool SB = D == 256;
  static constexpr int DQ_NAT = SB ? (MODE == BWD_DUAL ? 2 : 1) : (MODE == BWD_DUAL ? 4 : 2);
  static constexpr int DQ_TR = MODE == BWD_DUAL ? 2 : 1;
  static constexpr int DKV_NAT = SB ? 0 : (MODE == BWD_DUAL ? 4 : 2);
  static constexpr int DKV_TR = MODE == BWD_DUAL ? 4 : 2;
  static constexpr size_t DQ_LDS = (size_t)(DQ_NAT * N_ELEMS + DQ_TR * T_ELEMS) * sizeof(T);
  static constexpr size_t DKV_LDS = (size_t)(DKV_NAT * N_ELEMS + DKV_TR * T_ELEMS) * sizeof(T) + 5 * BWD_T * sizeof(float);
};

// whether the dq / dk,dv kernels fetch the next tile into registers during the current one's
// computation (needs up to 64 registers; see the forward kernel)
template <typename T, int D> constexpr bool BWD_FETCH_AHEAD = D == 64 || (D == 32 && sizeof(T) == 4);
// rows of 512 bytes: the resident operands of the dual backward fill the register file by themselves
template <typename T, int D> constexpr bool BWD_WIDE_ROWS = D * sizeof(T) >= 512;

template <int KK, typename T>
__device__ __forceinline__ void load_row_frags(Frag<T> *f, const T *row, int g) {
#pragma unroll
  for (int kk = 0; kk < KK; ++kk) f[kk] = ld8<T>(row + 16 * kk + 8 * g);
}

template <int KK, typename T>
__device__ __forceinline__ void gemm_tile(f32x16 &acc, const T *tile, int ld, int arow, int g, const Frag<T> *b) {
#pragma unroll
  for (int kk = 0; kk < KK; ++kk) {
    mma(acc, lds_frag(tile + arow * ld + 16 * kk + 8 * g), b[kk]);
    // rows of 512 bytes (fp32 D = 128): the register file is full of resident operands; keep the
    // scheduler from hoisting more than four fragment reads above the products that consume them
    if constexpr (KK * sizeof(Frag<T>) >= 256) {
      if (kk % 4 == 3) __builtin_amdgcn_sched_barrier(0);
    }
  }
}

// The same with the B fragments (the lane's own row) read from global memory where they are used; `tile` may
// be an LDS tile or rows of global memory (then `ld` is the row length and `arow` an index clamped by the caller).
template <int KK, typename T>
__device__ __forceinline__ void gemm_tile(f32x16 &acc, const T *tile, int ld, int arow, int g, const T *brow) {
#pragma unroll
  for (int kk = 0; kk < KK; ++kk) {
    mma(acc, lds_frag(tile + (size_t)arow * ld + 16 * kk + 8 * g), ld8<T>(brow + 16 * kk + 8 * g));
    if (kk % 4 == 3) __builtin_amdgcn_sched_barrier(0);
  }
}

__device__ __forceinline__ void zero16(f32x16 &x) {
#pragma unroll
  for (int e = 0; e < 16; ++e) x[e] = 0.f;
}

// ------------------------------------------------------------------------------------------------
// dq (MODE PLAIN / DUAL) or dq' (MODE TANGENT).  Scores are transposed (lane = query), as in the
// forward, so ds is already the B operand of dQ^T += K^T dS^T.
template <typename T, int D, int MODE, int MASK, bool DROP = false>
__global__ __launch_bounds__(256, 1) void bwd_dq_kernel(const BwdParams p) {
  using Cfg = BwdCfg<T, D, MODE>;
  constexpr int KK = D / 16, DB = D / 32;
  constexpr bool DUAL = MODE == BWD_DUAL, TAN = MODE == BWD_TANGENT;
  constexpr float NEG_INF = -__builtin_inff();

  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  constexpr bool SB = Cfg::SB;    // V, V' are not staged (see BwdCfg)
  T *Kn = reinterpret_cast<T *>(smem_raw);
  T *Vn = Kn + Cfg::N_ELEMS;
  T *KT = SB ? Vn : Vn + Cfg::N_ELEMS;
  T *Ktn = KT + Cfg::T_ELEMS;     // DUAL only from here on
  T *Vtn = Ktn + Cfg::N_ELEMS;
  T *KtT = SB ? Vtn : Vtn + Cfg::N_ELEMS;

  const Problem &pr = p.pr;
  const int L = pr.L;
  const int nqb = (L + BWD_BLK - 1) / BWD_BLK;
  const int total = nqb * pr.Z * pr.H;
  const int id = xcd_remap(blockIdx.x, nqb, pr.Z * pr.H);
  const int zh = id / nqb;
  const int qb = pr.causal ? nqb - 1 - id % nqb : id % nqb;
  const int z = zh / pr.H, h = zh % pr.H;
  const int tid = threadIdx.x, wave = tid / WAVE, lane = tid % WAVE;
  const int r = lane % 32, g = lane / 32, pr32 = perm32(r);

  const size_t head = (size_t)zh * L * D;
  const size_t srow = (size_t)zh * L;
  const int q0 = qb * BWD_BLK;
  const int qrow = q0 + wave * 32 + r;
  const int qld = qrow < L ? qrow : L - 1;
  const bool has_go = p.go != nullptr;

  // this lane's own row of the tensors that are B operands: resident fragments, or (SB) pointers to read through
  const T *Qrow = reinterpret_cast<const T *>(p.q) + head + (size_t)qld * D;
  const T *gOrow = (!TAN && has_go) ? reinterpret_cast<const T *>(p.go) + head + (size_t)qld * D : nullptr;
  const T *Qtrow = DUAL ? reinterpret_cast<const T *>(p.qt) + head + (size_t)qld * D : nullptr;
  const T *gTrow = (DUAL || TAN) ? reinterpret_cast<const T *>(p.gt) + head + (size_t)qld * D : nullptr;
  constexpr int KR = SB ? 1 : KK;
  Frag<T> Qf[KR], gOf[TAN ? 1 : KR], Qtf[DUAL ? KR : 1], gTf[(DUAL || TAN) ? KR : 1];
  if constexpr (!SB) {
    load_row_frags<KK>(Qf, Qrow, g);
    if constexpr (!TAN) {
      if (has_go) load_row_frags<KK>(gOf, gOrow, g);
    }
    if constexpr (DUAL) load_row_frags<KK>(Qtf, Qtrow, g);
    if constexpr (DUAL || TAN) load_row_frags<KK>(gTf, gTrow, g);
  }

  const float Mq = qrow < L ? p.M[srow + qld] : __builtin_inff();
  const float d1 = (MODE == BWD_PLAIN) ? p.d1[srow + qld] : 0.f;  // BWD_DUAL: d2 already holds d1 + d2
  const float mu = (DUAL) ? p.mu[srow + qld] : 0.f;
  const float av = (DUAL || TAN) ? p.a[srow + qld] : 0.f;
  const float d2 = (DUAL) ? p.d2[srow + qld] : 0.f;

  f32x16 acc[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db) zero16(acc[db]);

  const float sl2 = pr.scale * LOG2E;
  const int64_t mrow = MASK != MASK_NONE ? z * pr.ms[0] + h * pr.ms[1] + (int64_t)qld * pr.ms[2] : 0;
  const int Lk = pr.Lk;  // keys; L counts queries
  const size_t kvhead = ((size_t)z * pr.Hk + h / (pr.H / pr.Hk)) * Lk * D;  // grouped heads share K, V
  const T *Kg = reinterpret_cast<const T *>(p.k) + kvhead;
  const T *Vg = reinterpret_cast<const T *>(p.v) + kvhead;
  const T *Ktg = DUAL ? reinterpret_cast<const T *>(p.kt) + kvhead : nullptr;
  const T *Vtg = DUAL ? reinterpret_cast<const T *>(p.vt) + kvhead : nullptr;

  int kend = pr.causal ? min(Lk, q0 + BWD_BLK) : Lk;
  // key tiles visited: up to kend (the causal diagonal, or the caller's key limit of a padded batch), or the
  // caller's list of the tiles of this query block that hold an attended entry
  TileWalk<BWD_T> walk;
  {
    const int *tl = nullptr;
    if constexpr (MASK != MASK_NONE) {
      if (pr.klimit) kend = min(kend, max(pr.klimit[z], 1));
      if (pr.tiles_q) tl = pr.tiles_q + tile_list_offset_q(pr, z, h, qb);
    }
    walk.init(tl, 0, kend, Lk);
  }
  // The next tile is fetched into registers while this one is computed and written to LDS behind the
  // barrier that follows; K (, K') is fetched once and written both ways.  (See the forward kernel for
  // where this is left out.)
  constexpr bool AHEAD = BWD_FETCH_AHEAD<T, D>;
  QuadChunks<T, BWD_T, D, BWD_NT> rk, rkt;
  RowChunks<T, BWD_T, D, BWD_NT> rv, rvt;
  auto fetch_tile = [&](int j0) {
    const int nvalid = Lk - j0;
    fetch_quads(rk, Kg + (size_t)j0 * D, nvalid, tid);
    fetch_rows(rv, Vg + (size_t)j0 * D, nvalid, tid);
    if constexpr (DUAL) {
      fetch_quads(rkt, Ktg + (size_t)j0 * D, nvalid, tid);
      fetch_rows(rvt, Vtg + (size_t)j0 * D, nvalid, tid);
    }
  };
  if constexpr (AHEAD) {
    if (walk.n > 0) fetch_tile(walk.at(0));
  }
  for (int it = 0; it < walk.n; ++it) {
    const int j0 = walk.at(it);
    __syncthreads();
    if constexpr (AHEAD) {
      put_quads_rows(Kn, Cfg::LDN, rk, tid);
      put_quads_transposed(KT, Cfg::LDT, rk, tid);
      put_rows(Vn, Cfg::LDN, rv, tid);
      if constexpr (DUAL) {
        put_quads_rows(Ktn, Cfg::LDN, rkt, tid);
        put_quads_transposed(KtT, Cfg::LDT, rkt, tid);
        put_rows(Vtn, Cfg::LDN, rvt, tid);
      }
    } else {
      const int nvalid = Lk - j0;
      copy_rows<T, BWD_T, D, BWD_NT>(Kn, Cfg::LDN, Kg + (size_t)j0 * D, nvalid, tid);
      if constexpr (!SB) copy_rows<T, BWD_T, D, BWD_NT>(Vn, Cfg::LDN, Vg + (size_t)j0 * D, nvalid, tid);
      copy_rows_transposed<T, BWD_T, D, BWD_NT>(KT, Cfg::LDT, Kg + (size_t)j0 * D, nvalid, tid);
      if constexpr (DUAL) {
        copy_rows<T, BWD_T, D, BWD_NT>(Ktn, Cfg::LDN, Ktg + (size_t)j0 * D, nvalid, tid);
        if constexpr (!SB) copy_rows<T, BWD_T, D, BWD_NT>(Vtn, Cfg::LDN, Vtg + (size_t)j0 * D, nvalid, tid);
        copy_rows_transposed<T, BWD_T, D, BWD_NT>(KtT, Cfg::LDT, Ktg + (size_t)j0 * D, nvalid, tid);
      }
    }
    __syncthreads();
    if constexpr (AHEAD) {
      if (it + 1 < walk.n) fetch_tile(walk.at(it + 1));
    }

    f32x16 S, dP, Sp, At;  // DUAL: dP also collects gT V'^T (the B term)
    zero16(S);
    if constexpr (SB) {
      // V, V' fragments from global memory: this lane's key row, clamped (a key past the end has p = 0 and
      // must meet finite values)
      const int vrow = min(j0 + pr32, Lk - 1);
      gemm_tile<KK>(S, Kn, Cfg::LDN, pr32, g, Qrow);
      if constexpr (!TAN) {
        zero16(dP);
        if (has_go) gemm_tile<KK>(dP, Vg, D, vrow, g, gOrow);
      }
      if constexpr (DUAL) {
        zero16(Sp);
        gemm_tile<KK>(Sp, Kn, Cfg::LDN, pr32, g, Qtrow);
        gemm_tile<KK>(Sp, Ktn, Cfg::LDN, pr32, g, Qrow);
        gemm_tile<KK>(dP, Vtg, D, vrow, g, gTrow);
      }
      if constexpr (DUAL || TAN) {
        zero16(At);
        gemm_tile<KK>(At, Vg, D, vrow, g, gTrow);
      }
    } else {
    gemm_tile<KK>(S, Kn, Cfg::LDN, pr32, g, Qf);
    if constexpr (!TAN) {
      zero16(dP);
      if (has_go) gemm_tile<KK>(dP, Vn, Cfg::LDN, pr32, g, gOf);
    }
    if constexpr (DUAL) {
      zero16(Sp);
      gemm_tile<KK>(Sp, Kn, Cfg::LDN, pr32, g, Qtf);
      gemm_tile<KK>(Sp, Ktn, Cfg::LDN, pr32, g, Qf);
      gemm_tile<KK>(dP, Vtn, Cfg::LDN, pr32, g, gTf);
    }
    if constexpr (DUAL || TAN) {
      zero16(At);
      gemm_tile<KK>(At, Vn, Cfg::LDN, pr32, g, gTf);
    }
    }

    const bool diag = pr.causal && (j0 + BWD_T - 1 > q0 + wave * 32);
    const bool ragged = j0 + BWD_T > Lk;
#pragma unroll
    for (int hf = 0; hf < 2; ++hf) {
      const int key0 = j0 + 16 * hf + 8 * g;
      float bias[8];
      bool keep[8];
      if constexpr (MASK == MASK_ADD) mask_bias8<T>(pr, mrow, key0, bias);
      if constexpr (MASK == MASK_BOOL) mask_keep8(pr, mrow, key0, keep);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int i = 8 * hf + e;
        float s = S[i] * sl2;
        if constexpr (MASK == MASK_ADD) s += bias[e];
        float pv = fast_exp2(s - Mq);
        if constexpr (MASK == MASK_BOOL) pv = keep[e] ? pv : 0.f;
        if (diag) pv = (key0 + e <= qrow) ? pv : 0.f;
        if (ragged) pv = (key0 + e < Lk) ? pv : 0.f;
        if constexpr (DROP) {  // gO V^T, gT V^T, gT V'^T reach the logits through the kept, rescaled entries only
          const float ks = drop_scale(pr, zh, qld, key0 + e);
          if constexpr (!TAN) dP[i] *= ks;
          if constexpr (DUAL || TAN) At[i] *= ks;
        }
        if constexpr (MODE == BWD_PLAIN) {
          S[i] = pv * (dP[i] - d1);
        } else if constexpr (DUAL) {
          const float sp = Sp[i] * pr.scale;
          Sp[i] = pv * (At[i] - av);
          S[i] = pv * (dP[i] - d1 + At[i] * (sp - mu) - av * sp - d2);
        } else {
          S[i] = pv * (At[i] - av);
        }
      }
    }

#pragma unroll
    for (int c = 0; c < BWD_T / 16; ++c) {
      Frag<T> dsf = to_frag<T>(S, c);
      Frag<T> dspf;
      if constexpr (DUAL) dspf = to_frag<T>(Sp, c);
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        mma(acc[db], lds_frag(KT + (32 * db + pr32) * Cfg::LDT + 16 * c + 8 * g), dsf);
        if constexpr (DUAL) mma(acc[db], lds_frag(KtT + (32 * db + pr32) * Cfg::LDT + 16 * c + 8 * g), dspf);
        if constexpr (BWD_WIDE_ROWS<T, D>) {  // as in gemm_tile, bound the fragment reads in flight
          if (db % 2 == 1) __builtin_amdgcn_sched_barrier(0);
        }
      }
    }
  }

  if (qrow < L) {
    T *out = reinterpret_cast<T *>(TAN ? p.dqt : p.dq) + head + (size_t)qrow * D;
#pragma unroll
    for (int db = 0; db < DB; ++db) {
#pragma unroll
      for (int hf = 0; hf < 2; ++hf) {
        float x[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) x[e] = acc[db][8 * hf + e] * pr.scale;
        store8<T>(out + 32 * db + 16 * hf + 8 * g, x);
      }
    }
  }
}

// ------------------------------------------------------------------------------------------------
// dk, dv (MODE PLAIN / DUAL) or dk', dv' (MODE TANGENT).  Scores are S = Q K^T (lane = key,
// registers = queries), so P and dS are the B operands of dV^T += gO^T P and dK^T += Q^T dS.
template <typename T, int D, int MODE, int MASK, bool DROP = false>
__global__ __launch_bounds__(256, 1) void bwd_dkdv_kernel(const BwdParams p) {
  using Cfg = BwdCfg<T, D, MODE>;
  constexpr int KK = D / 16, DB = D / 32;
  constexpr bool DUAL = MODE == BWD_DUAL, TAN = MODE == BWD_TANGENT;

  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  // row-major tiles first, then transposed ones, then the row statistics
  T *Qn = reinterpret_cast<T *>(smem_raw);
  T *Gn = Qn + Cfg::N_ELEMS;                         // gO (PLAIN, DUAL) or gT (TANGENT)
  T *Qtn = Gn + Cfg::N_ELEMS;                        // DUAL: Q'
  T *GTn = Qtn + Cfg::N_ELEMS;                       // DUAL: gT
  T *trbase = Qn + Cfg::DKV_NAT * Cfg::N_ELEMS;
  T *QT = trbase;
  T *GT = QT + Cfg::T_ELEMS;
  T *QtT = GT + Cfg::T_ELEMS;                        // DUAL
  T *GTT = QtT + Cfg::T_ELEMS;                       // DUAL
  float *stats = reinterpret_cast<float *>(trbase + Cfg::DKV_TR * Cfg::T_ELEMS);
  float *sM = stats, *sd1 = stats + BWD_T, *smu = stats + 2 * BWD_T, *sa = stats + 3 * BWD_T, *sd2 = stats + 4 * BWD_T;

  // One workgroup per (batch entry, key/value head, block of 128 keys).  With grouped heads the query
  // heads of the group are visited one after another and their contributions add up in dK, dV.
  const Problem &pr = p.pr;
  const int L = pr.L, Lk = pr.Lk;  // queries, keys
  const int nkb = (Lk + BWD_BLK - 1) / BWD_BLK;
  const int id = xcd_remap(blockIdx.x, nkb, pr.Z * pr.Hk);
  const int zhk = id / nkb;
  const int kb = id % nkb;  // causal: the first key blocks have the longest query loops
  const int z = zhk / pr.Hk, hk = zhk % pr.Hk, group = pr.H / pr.Hk;
  const int tid = threadIdx.x, wave = tid / WAVE, lane = tid % WAVE;
  const int r = lane % 32, g = lane / 32, pr32 = perm32(r);

  const size_t kvhead = (size_t)zhk * Lk * D;
  const int k0 = kb * BWD_BLK;
  const int krow = k0 + wave * 32 + r;
  const int kld = krow < Lk ? krow : Lk - 1;
  const bool has_go = p.go != nullptr;

  // this lane's own key row of K, V (, K', V'): resident fragments, or (SB, see BwdCfg) pointers to read through
  constexpr bool SB = Cfg::SB;
  const T *Krow = reinterpret_cast<const T *>(p.k) + kvhead + (size_t)kld * D;
  const T *Vrow = reinterpret_cast<const T *>(p.v) + kvhead + (size_t)kld * D;
  const T *Ktrow = DUAL ? reinterpret_cast<const T *>(p.kt) + kvhead + (size_t)kld * D : nullptr;
  const T *Vtrow = DUAL ? reinterpret_cast<const T *>(p.vt) + kvhead + (size_t)kld * D : nullptr;
  constexpr int KR = SB ? 1 : KK;
  Frag<T> Kf[KR], Vf[KR], Ktf[DUAL ? KR : 1], Vtf[DUAL ? KR : 1];
  if constexpr (!SB) {
    load_row_frags<KK>(Kf, Krow, g);
    load_row_frags<KK>(Vf, Vrow, g);
    if constexpr (DUAL) {
      load_row_frags<KK>(Ktf, Ktrow, g);
      load_row_frags<KK>(Vtf, Vtrow, g);
    }
  }

  f32x16 dK[DB], dV[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db) {
    zero16(dK[db]);
    zero16(dV[db]);
  }

  const float sl2 = pr.scale * LOG2E;
  const int istart = pr.causal ? (k0 / BWD_T) * BWD_T : 0;
  for (int gi = 0; gi < group; ++gi) {
  const int h = hk * group + gi;  // query head
  const size_t head = ((size_t)z * pr.H + h) * L * D;
  const size_t srow = ((size_t)z * pr.H + h) * L;
  const T *Qg = reinterpret_cast<const T *>(p.q) + head;
  const T *Qtg = DUAL ? reinterpret_cast<const T *>(p.qt) + head : nullptr;
  const T *gOg = (!TAN && has_go) ? reinterpret_cast<const T *>(p.go) + head : nullptr;
  const T *gTg = (DUAL || TAN) ? reinterpret_cast<const T *>(p.gt) + head : nullptr;
  const T *Gg = TAN ? gTg : gOg;  // tensor staged in Gn / GT
  // The next tile (each tensor once, written to LDS both ways) and its row statistics are fetched
  // into registers while this tile is computed, as in the dq kernel.
  constexpr bool AHEAD = BWD_FETCH_AHEAD<T, D>;
  QuadChunks<T, BWD_T, D, BWD_NT> rq, rg, rqt, rgt;
  float rs[5] = {0.f, 0.f, 0.f, 0.f, 0.f};  // M, d1, mu, a, d2 of query row i0 + tid
  auto fetch_stats = [&](int i0) {
    if (tid < BWD_T) {
      const bool ok = i0 + tid < L;
      const size_t si = srow + (ok ? i0 + tid : 0);
      rs[0] = ok ? p.M[si] : __builtin_inff();
      rs[1] = (ok && MODE == BWD_PLAIN) ? p.d1[si] : 0.f;  // BWD_DUAL: d2 already holds d1 + d2
      rs[2] = (ok && DUAL) ? p.mu[si] : 0.f;
      rs[3] = (ok && (DUAL || TAN)) ? p.a[si] : 0.f;
      rs[4] = (ok && DUAL) ? p.d2[si] : 0.f;
    }
  };
  auto put_stats = [&]() {
    if (tid < BWD_T) {
      sM[tid] = rs[0], sd1[tid] = rs[1], smu[tid] = rs[2], sa[tid] = rs[3], sd2[tid] = rs[4];
    }
  };
  auto fetch_tile = [&](int i0) {
    const int nvalid = L - i0;
    fetch_quads(rq, Qg + (size_t)i0 * D, nvalid, tid);
    if (Gg) fetch_quads(rg, Gg + (size_t)i0 * D, nvalid, tid);
    if constexpr (DUAL) {
      fetch_quads(rqt, Qtg + (size_t)i0 * D, nvalid, tid);
      fetch_quads(rgt, gTg + (size_t)i0 * D, nvalid, tid);
    }
    fetch_stats(i0);
  };
  // query tiles visited: all from istart on, or the caller's list of the tiles of this key block (and this
  // query head's mask plane) that hold an attended entry
  TileWalk<BWD_T> walk;
  {
    const int *tl = nullptr;
    if constexpr (MASK != MASK_NONE) {
      if (pr.tiles_k) tl = pr.tiles_k + tile_list_offset_k(pr, z, h, kb);
    }
    walk.init(tl, istart, L, L);
    if constexpr (MASK != MASK_NONE) {
      if (pr.klimit && k0 >= pr.klimit[z]) walk.n = 0;  // a key block the caller's hint declares fully masked: zeros
    }
  }
  if constexpr (AHEAD) {
    if (walk.n > 0) fetch_tile(walk.at(0));
  }
  for (int it = 0; it < walk.n; ++it) {
    const int i0 = walk.at(it);
    __syncthreads();
    if constexpr (AHEAD) {
      put_quads_rows(Qn, Cfg::LDN, rq, tid);
      put_quads_transposed(QT, Cfg::LDT, rq, tid);
      if (Gg) {
        put_quads_rows(Gn, Cfg::LDN, rg, tid);
        put_quads_transposed(GT, Cfg::LDT, rg, tid);
      }
      if constexpr (DUAL) {
        put_quads_rows(Qtn, Cfg::LDN, rqt, tid);
        put_quads_transposed(QtT, Cfg::LDT, rqt, tid);
        put_quads_rows(GTn, Cfg::LDN, rgt, tid);
        put_quads_transposed(GTT, Cfg::LDT, rgt, tid);
      }
    } else {
      const int nvalid = L - i0;
      if constexpr (!SB) copy_rows<T, BWD_T, D, BWD_NT>(Qn, Cfg::LDN, Qg + (size_t)i0 * D, nvalid, tid);
      copy_rows_transposed<T, BWD_T, D, BWD_NT>(QT, Cfg::LDT, Qg + (size_t)i0 * D, nvalid, tid);
      if (Gg) {
        if constexpr (!SB) copy_rows<T, BWD_T, D, BWD_NT>(Gn, Cfg::LDN, Gg + (size_t)i0 * D, nvalid, tid);
        copy_rows_transposed<T, BWD_T, D, BWD_NT>(GT, Cfg::LDT, Gg + (size_t)i0 * D, nvalid, tid);
      }
      if constexpr (DUAL) {
        if constexpr (!SB) copy_rows<T, BWD_T, D, BWD_NT>(Qtn, Cfg::LDN, Qtg + (size_t)i0 * D, nvalid, tid);
        copy_rows_transposed<T, BWD_T, D, BWD_NT>(QtT, Cfg::LDT, Qtg + (size_t)i0 * D, nvalid, tid);
        if constexpr (!SB) copy_rows<T, BWD_T, D, BWD_NT>(GTn, Cfg::LDN, gTg + (size_t)i0 * D, nvalid, tid);
        copy_rows_transposed<T, BWD_T, D, BWD_NT>(GTT, Cfg::LDT, gTg + (size_t)i0 * D, nvalid, tid);
      }
      fetch_stats(i0);
    }
    put_stats();
    __syncthreads();
    if constexpr (AHEAD) {
      if (it + 1 < walk.n) fetch_tile(walk.at(it + 1));
    }

    f32x16 S, dP, Sp, At;  // DUAL: dP also collects V' gT^T (the B term)
    zero16(S);
    if constexpr (SB) {
      // row-wise fragments of Q, G (, Q', gT) from global memory: this lane's query row, clamped (a query past
      // the end has p = 0 and must meet finite values)
      const int qr = min(i0 + pr32, L - 1);
      gemm_tile<KK>(S, Qg, D, qr, g, Krow);
      if constexpr (!TAN) {
        zero16(dP);
        if (has_go) gemm_tile<KK>(dP, Gg, D, qr, g, Vrow);
      }
      if constexpr (DUAL) {
        zero16(Sp);
        gemm_tile<KK>(Sp, Qtg, D, qr, g, Krow);
        gemm_tile<KK>(Sp, Qg, D, qr, g, Ktrow);
        zero16(At);
        gemm_tile<KK>(At, gTg, D, qr, g, Vrow);
        gemm_tile<KK>(dP, gTg, D, qr, g, Vtrow);
      }
      if constexpr (TAN) {
        zero16(At);
        gemm_tile<KK>(At, Gg, D, qr, g, Vrow);
      }
    } else {
    gemm_tile<KK>(S, Qn, Cfg::LDN, pr32, g, Kf);
    if constexpr (!TAN) {
      zero16(dP);
      if (has_go) gemm_tile<KK>(dP, Gn, Cfg::LDN, pr32, g, Vf);
    }
    if constexpr (DUAL) {
      zero16(Sp);
      gemm_tile<KK>(Sp, Qtn, Cfg::LDN, pr32, g, Kf);
      gemm_tile<KK>(Sp, Qn, Cfg::LDN, pr32, g, Ktf);
      zero16(At);
      gemm_tile<KK>(At, GTn, Cfg::LDN, pr32, g, Vf);
      gemm_tile<KK>(dP, GTn, Cfg::LDN, pr32, g, Vtf);
    }
    if constexpr (TAN) {
      zero16(At);
      gemm_tile<KK>(At, Gn, Cfg::LDN, pr32, g, Vf);
    }
    }

    const bool diag = pr.causal && (i0 < k0 + wave * 32 + 31);  // some query may precede a key
    f32x16 Pp;  // DUAL: P*(S'-mu); TANGENT: unused
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const int ql = 16 * (e / 8) + 8 * g + (e % 8);  // query row within the tile
      const int qi = i0 + ql;
      float s = S[e] * sl2;
      bool keep = true;
      if constexpr (MASK != MASK_NONE) {
        const int qc = qi < L ? qi : L - 1;
        const int64_t off = z * pr.ms[0] + h * pr.ms[1] + (int64_t)qc * pr.ms[2] + (int64_t)kld * pr.ms[3];
        if constexpr (MASK == MASK_ADD) s += (float)reinterpret_cast<const T *>(pr.mask)[off] * LOG2E;
        if constexpr (MASK == MASK_BOOL) keep = reinterpret_cast<const uint8_t *>(pr.mask)[off] != 0;
      }
      float pv = fast_exp2(s - sM[ql]);
      if constexpr (MASK == MASK_BOOL) pv = keep ? pv : 0.f;
      if (diag) pv = (krow <= qi) ? pv : 0.f;
      float ks = 1.f;  // dropout: 1 / (1 - p) for a kept entry, 0 for a dropped one
      if constexpr (DROP) {
        ks = drop_scale(pr, z * pr.H + h, qi < L ? qi : L - 1, kld);
        if constexpr (!TAN) dP[e] *= ks;
        if constexpr (DUAL || TAN) At[e] *= ks;
      }
      if constexpr (MODE == BWD_PLAIN) {
        S[e] = pv * ks;
        dP[e] = pv * (dP[e] - sd1[ql]);
      } else if constexpr (DUAL) {
        const float sp = Sp[e] * pr.scale, m_ = smu[ql], a_ = sa[ql];
        S[e] = pv * ks;
        Pp[e] = pv * (sp - m_) * ks;
        Sp[e] = pv * (At[e] - a_);
        dP[e] = pv * (dP[e] - sd1[ql] + At[e] * (sp - m_) - a_ * sp - sd2[ql]);
      } else {
        S[e] = pv * ks;
        Sp[e] = pv * (At[e] - sa[ql]);
      }
    }

#pragma unroll
    for (int c = 0; c < BWD_T / 16; ++c) {
      Frag<T> pf = to_frag<T>(S, c);
      Frag<T> dsf, dspf, ppf;
      if constexpr (!TAN) dsf = to_frag<T>(dP, c);
      if constexpr (DUAL || TAN) dspf = to_frag<T>(Sp, c);
      if constexpr (DUAL) ppf = to_frag<T>(Pp, c);
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        const int off = (32 * db + pr32) * Cfg::LDT + 16 * c + 8 * g;
        if constexpr (MODE == BWD_PLAIN) {
          mma(dK[db], lds_frag(QT + off), dsf);
          mma(dV[db], lds_frag(GT + off), pf);
        } else if constexpr (DUAL) {
          mma(dK[db], lds_frag(QT + off), dsf);
          mma(dK[db], lds_frag(QtT + off), dspf);
          if (has_go) mma(dV[db], lds_frag(GT + off), pf);
          mma(dV[db], lds_frag(GTT + off), ppf);
        } else {
          mma(dK[db], lds_frag(QT + off), dspf);
          mma(dV[db], lds_frag(GT + off), pf);
        }
        if constexpr (BWD_WIDE_ROWS<T, D>) {  // as in gemm_tile, bound the fragment reads in flight
          if (db % 2 == 1) __builtin_amdgcn_sched_barrier(0);
        }
      }
    }
  }
  }  // query heads of the group

  if (krow < Lk) {
    T *outk = reinterpret_cast<T *>(TAN ? p.dkt : p.dk) + kvhead + (size_t)krow * D;
    T *outv = reinterpret_cast<T *>(TAN ? p.dvt : p.dv) + kvhead + (size_t)krow * D;
#pragma unroll
    for (int db = 0; db < DB; ++db) {
#pragma unroll
      for (int hf = 0; hf < 2; ++hf) {
        float xk[8], xv[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          xk[e] = dK[db][8 * hf + e] * pr.scale;
          xv[e] = dV[db][8 * hf + e];
        }
        store8<T>(outk + 32 * db + 16 * hf + 8 * g, xk);
        store8<T>(outv + 32 * db + 16 * hf + 8 * g, xv);
      }
    }
  }
}

}  // namespace jvpfa
