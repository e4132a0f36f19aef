// Fused dual forward: O, O', M, mu in one pass over LDS-staged K/K'/V/V' tiles.
//
// Work split: one workgroup of 4 waves owns 128 query rows of one (z, h); each wave owns 32
// of them and keeps Q, Q' (B operands) and the accumulators O^T, T^T (D x 32 each) in
// registers.  Scores are formed transposed, S^T = K Q^T, so that a lane owns one query column:
// the running max / sum / mu are per-lane scalars (one cross-half exchange per tile) and the
// probabilities are already laid out as the B operand of O^T += V^T P^T.
//
// Replaces the reference's _attn_fwd / _attn_fwd_inner (jvp_attention.py:662-1033, :125-336);
// its three accumulators acc, g_acc, p_tv_acc (:872, :916-918) become two, O and
// T = sum((p*s')V + pV'), since g_acc and p_tv_acc share every rescale and are only summed
// (:1031-1033).
#pragma once
#include "common.hpp"
#include "mask.hpp"
#include "params.hpp"

namespace jvpfa {

template <typename T, int D, int BN, bool DUAL> struct FwdCfg {
  static constexpr int NW = 4;
  static constexpr int NT = NW * WAVE;
  static constexpr int BM = NW * 32;
  static constexpr int PAD = 16 / sizeof(T);
  static constexpr int LDK = D + PAD;   // row stride of the row-major K tiles
  static constexpr int LDV = BN + PAD;  // row stride of the transposed V tiles
  static constexpr int K_ELEMS = BN * LDK;
  static constexpr int V_ELEMS = D * LDV;
  static constexpr size_t LDS_BYTES = (size_t)(DUAL ? 2 : 1) * (K_ELEMS + V_ELEMS) * sizeof(T);
};

// DROP: dropout on the probabilities (the row sums l, mu stay those of the full softmax; what enters the
// products with V, V' is P * keep / (1 - p)).  The reference has dead code for it and raises (its
// jvp_attention.py:94-122, :271-277, :2356-2357).
template <typename T, int D, int BN, bool DUAL, int MASK, bool DROP = false>
__global__ __launch_bounds__(256, 1) void fwd_kernel(const FwdParams p) {
  using Cfg = FwdCfg<T, D, BN, DUAL>;
  constexpr int NB = BN / 32;  // 32-key score blocks per tile
  constexpr int KK = D / 16;   // contraction steps over the head dimension
  constexpr int DB = D / 32;   // 32-row blocks of the transposed outputs
  constexpr float NEG_INF = -__builtin_inff();

  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  T *Ks = reinterpret_cast<T *>(smem_raw);
  T *Vs = Ks + Cfg::K_ELEMS;
  T *Kts = Vs + Cfg::V_ELEMS;   // K' (only when DUAL)
  T *Vts = Kts + Cfg::K_ELEMS;  // V'

  const Problem &pr = p.pr;
  const int L = pr.L;
  const int nqb = (L + Cfg::BM - 1) / Cfg::BM;
  const int total = nqb * pr.Z * pr.H;
  const int id = xcd_remap(blockIdx.x, nqb, pr.Z * pr.H);
  const int zh = id / nqb;
  // causal: the last query blocks have the longest key loops, start them first
  const int qb = pr.causal ? nqb - 1 - id % nqb : id % nqb;
  const int z = zh / pr.H, h = zh % pr.H;

  const int tid = threadIdx.x;
  const int wave = tid / WAVE, lane = tid % WAVE;
  const int r = lane % 32, g = lane / 32;
  const int pr32 = perm32(r);

  const int Lk = pr.Lk;  // keys; L counts queries
  const size_t head = (size_t)zh * L * D;
  const size_t kvhead = ((size_t)z * pr.Hk + h / (pr.H / pr.Hk)) * Lk * D;  // grouped heads share K, V
  const T *Qg = reinterpret_cast<const T *>(p.q) + head;
  const T *Kg = reinterpret_cast<const T *>(p.k) + kvhead;
  const T *Vg = reinterpret_cast<const T *>(p.v) + kvhead;
  const T *Qtg = DUAL ? reinterpret_cast<const T *>(p.qt) + head : nullptr;
  const T *Ktg = DUAL ? reinterpret_cast<const T *>(p.kt) + kvhead : nullptr;
  const T *Vtg = DUAL ? reinterpret_cast<const T *>(p.vt) + kvhead : nullptr;

  const int q0 = qb * Cfg::BM;         // first query row of the workgroup
  const int qrow = q0 + wave * 32 + r; // this lane's query row
  const int qld = qrow < L ? qrow : L - 1;

  // D = 256 (fp32 only: the 16-bit types have kernels of their own at this head dim, fwd_kernel_wide.hpp): Q, Q'
  // resident would be up to 256 registers next to 256 of accumulators, so there the lane's fragments are read
  // from global memory where they are used (the same 32 bytes per lane on every tile: cache hits)
  constexpr bool SB = D == 256;
  const T *Qrow = Qg + (size_t)qld * D + 8 * g, *Qtrow = DUAL ? Qtg + (size_t)qld * D + 8 * g : nullptr;
  Frag<T> Qf[SB ? 1 : KK], Qtf[(DUAL && !SB) ? KK : 1];
  if constexpr (!SB) {
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
      Qf[kk] = ld8<T>(Qrow + 16 * kk);
      if constexpr (DUAL) Qtf[kk] = ld8<T>(Qtrow + 16 * kk);
    }
  }

  f32x16 Oacc[DB], Tacc[DUAL ? DB : 1];
#pragma unroll
  for (int db = 0; db < DB; ++db) {
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      Oacc[db][e] = 0.f;
      if constexpr (DUAL) Tacc[db][e] = 0.f;
    }
  }
  float m_i = NEG_INF, l_i = 0.f, mu_i = 0.f;  // l_i, mu_i: partial over this lane's keys

  const float sl2 = pr.scale * LOG2E;
  const int64_t mrow = MASK != MASK_NONE ? z * pr.ms[0] + h * pr.ms[1] + (int64_t)qld * pr.ms[2] : 0;

  int kend = Lk;
  if (pr.causal) kend = min(Lk, q0 + Cfg::BM);
  // key tiles visited: up to kend (the causal diagonal, or the caller's key limit of a padded batch), or the
  // caller's list of the tiles of this query block that hold an attended entry
  TileWalk<BN> walk;
  {
    const int *tl = nullptr;
    if constexpr (MASK != MASK_NONE) {
      if (pr.klimit) kend = min(kend, max(pr.klimit[z], 1));
      if (pr.tiles_q) tl = pr.tiles_q + tile_list_offset_q(pr, z, h, qb);
    }
    walk.init(tl, 0, kend, Lk);
  }

  // The next tile is fetched into registers while this one is computed and written to LDS behind the
  // barrier that follows.  Not for D >= 128 (no registers to spare) and not for 16-bit D = 32, where
  // the registers would cost the second and third workgroup per compute unit that hide the latency
  // better (403 vs 327 TFLOP/s measured).
  constexpr bool AHEAD = D == 64 || (D == 32 && sizeof(T) == 4);
  RowChunks<T, BN, D, Cfg::NT> rk, rkt;
  QuadChunks<T, BN, D, Cfg::NT> rv, rvt;
  auto fetch_tile = [&](int j0) {
    const int nvalid = Lk - j0;  // rows >= nvalid are zero-filled
    fetch_rows(rk, Kg + (size_t)j0 * D, nvalid, tid);
    fetch_quads(rv, Vg + (size_t)j0 * D, nvalid, tid);
    if constexpr (DUAL) {
      fetch_rows(rkt, Ktg + (size_t)j0 * D, nvalid, tid);
      fetch_quads(rvt, Vtg + (size_t)j0 * D, nvalid, tid);
    }
  };
  if constexpr (AHEAD) {
    if (walk.n > 0) fetch_tile(walk.at(0));
  }
  for (int it = 0; it < walk.n; ++it) {
    const int j0 = walk.at(it);
    __syncthreads();
    if constexpr (AHEAD) {
      put_rows(Ks, Cfg::LDK, rk, tid);
      put_quads_transposed(Vs, Cfg::LDV, rv, tid);
      if constexpr (DUAL) {
        put_rows(Kts, Cfg::LDK, rkt, tid);
        put_quads_transposed(Vts, Cfg::LDV, rvt, tid);
      }
    } else {
      const int nvalid = Lk - j0;  // rows >= nvalid are zero-filled
      copy_rows<T, BN, D, Cfg::NT>(Ks, Cfg::LDK, Kg + (size_t)j0 * D, nvalid, tid);
      copy_rows_transposed<T, BN, D, Cfg::NT>(Vs, Cfg::LDV, Vg + (size_t)j0 * D, nvalid, tid);
      if constexpr (DUAL) {
        copy_rows<T, BN, D, Cfg::NT>(Kts, Cfg::LDK, Ktg + (size_t)j0 * D, nvalid, tid);
        copy_rows_transposed<T, BN, D, Cfg::NT>(Vts, Cfg::LDV, Vtg + (size_t)j0 * D, nvalid, tid);
      }
    }
    __syncthreads();
    if constexpr (AHEAD) {
      if (it + 1 < walk.n) fetch_tile(walk.at(it + 1));
    }

    // ---- S^T = K Q^T and S'^T = K Q'^T + K' Q^T -------------------------------------------
    f32x16 S[NB], Sp[DUAL ? NB : 1];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        S[nb][e] = 0.f;
        if constexpr (DUAL) Sp[nb][e] = 0.f;
      }
#pragma unroll
      for (int kk = 0; kk < KK; ++kk) {
        Frag<T> a = lds_frag(Ks + (32 * nb + pr32) * Cfg::LDK + 16 * kk + 8 * g);
        if constexpr (SB) {
          const Frag<T> qf = ld8<T>(Qrow + 16 * kk);
          mma(S[nb], a, qf);
          if constexpr (DUAL) {
            mma(Sp[nb], a, ld8<T>(Qtrow + 16 * kk));
            Frag<T> a2 = lds_frag(Kts + (32 * nb + pr32) * Cfg::LDK + 16 * kk + 8 * g);
            mma(Sp[nb], a2, qf);
          }
          if (kk % 4 == 3) __builtin_amdgcn_sched_barrier(0);  // bound the fragment reads in flight
        } else {
        mma(S[nb], a, Qf[kk]);
        if constexpr (DUAL) {
          mma(Sp[nb], a, Qtf[kk]);
          Frag<T> a2 = lds_frag(Kts + (32 * nb + pr32) * Cfg::LDK + 16 * kk + 8 * g);
          mma(Sp[nb], a2, Qf[kk]);
        }
        }
      }
    }

    // ---- online softmax in the log2 domain (per-lane query column) -------------------------
    const bool diag = pr.causal && (j0 + BN - 1 > q0 + wave * 32);  // some key may exceed a query
    const bool ragged = j0 + BN > Lk;
    float mx = NEG_INF;
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
#pragma unroll
      for (int hf = 0; hf < 2; ++hf) {
        const int key0 = j0 + 32 * nb + 16 * hf + 8 * g;
        float bias[8];
        bool keep[8];
        if constexpr (MASK == MASK_ADD) mask_bias8<T>(pr, mrow, key0, bias);
        if constexpr (MASK == MASK_BOOL) mask_keep8(pr, mrow, key0, keep);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          float s = S[nb][8 * hf + e] * sl2;
          if constexpr (MASK == MASK_ADD) s += bias[e];
          if constexpr (MASK == MASK_BOOL) s = keep[e] ? s : NEG_INF;
          if (diag) s = (key0 + e <= qrow) ? s : NEG_INF;
          if (ragged) s = (key0 + e < Lk) ? s : NEG_INF;
          S[nb][8 * hf + e] = s;
          mx = fmaxf(mx, s);
        }
      }
    }
    mx = fmaxf(mx, xor32(mx));
    const float m_new = fmaxf(m_i, mx);
    const float m_use = (m_new == NEG_INF) ? 0.f : m_new;
    const float alpha = fast_exp2(m_i - m_use);
    float rs = 0.f, rmu = 0.f;
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        float pv = fast_exp2(S[nb][e] - m_use);
        rs += pv;
        float ks = 1.f;
        if constexpr (DROP) {
          const int key = j0 + 32 * nb + 16 * (e / 8) + 8 * g + (e % 8);
          ks = drop_scale(pr, zh, qld, key);
        }
        S[nb][e] = pv * ks;
        if constexpr (DUAL) {
          float ps = pv * (Sp[nb][e] * pr.scale);
          rmu += ps;
          Sp[nb][e] = ps * ks;
        }
      }
    }
    l_i = l_i * alpha + rs;
    m_i = m_new;
    if constexpr (DUAL) mu_i = mu_i * alpha + rmu;
#pragma unroll
    for (int db = 0; db < DB; ++db) {
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        Oacc[db][e] *= alpha;
        if constexpr (DUAL) Tacc[db][e] *= alpha;
      }
    }

    // ---- O^T += V^T P^T,  T^T += V^T (P*S')^T + V'^T P^T -----------------------------------
#pragma unroll
    for (int c = 0; c < BN / 16; ++c) {
      Frag<T> pf = to_frag<T>(S[c / 2], c % 2);
      Frag<T> psf;
      if constexpr (DUAL) psf = to_frag<T>(Sp[c / 2], c % 2);
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        Frag<T> a = lds_frag(Vs + (32 * db + pr32) * Cfg::LDV + 16 * c + 8 * g);
        mma(Oacc[db], a, pf);
        if constexpr (DUAL) {
          mma(Tacc[db], a, psf);
          Frag<T> a2 = lds_frag(Vts + (32 * db + pr32) * Cfg::LDV + 16 * c + 8 * g);
          mma(Tacc[db], a2, pf);
        }
      }
    }
  }

  // ---- epilogue (reference jvp_attention.py:1010-1033) ---------------------------------------
  l_i += xor32(l_i);
  if constexpr (DUAL) mu_i += xor32(mu_i);
  const bool dead = !(l_i > 0.f);
  const float inv = dead ? 0.f : 1.f / l_i;
  const float mu_n = mu_i * inv;
  if (qrow < L) {
    T *Og = reinterpret_cast<T *>(p.o) + head + (size_t)qrow * D;
    T *Otg = DUAL ? reinterpret_cast<T *>(p.ot) + head + (size_t)qrow * D : nullptr;
#pragma unroll
    for (int db = 0; db < DB; ++db) {
#pragma unroll
      for (int hf = 0; hf < 2; ++hf) {
        float o8[8], t8[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          o8[e] = Oacc[db][8 * hf + e] * inv;
          if constexpr (DUAL) t8[e] = Tacc[db][8 * hf + e] * inv - mu_n * o8[e];
        }
        const int d0 = 32 * db + 16 * hf + 8 * g;
        store8<T>(Og + d0, o8);
        if constexpr (DUAL) store8<T>(Otg + d0, t8);
      }
    }
    if (g == 0) {
      p.M[(size_t)zh * L + qrow] = dead ? __builtin_inff() : m_i + __builtin_amdgcn_logf(l_i);
      if constexpr (DUAL) p.mu[(size_t)zh * L + qrow] = mu_n;
    }
  }
}

}  // namespace jvpfa
