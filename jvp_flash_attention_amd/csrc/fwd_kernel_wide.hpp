// Forward for 16-bit element types with D = 256.
//
// With D = 256 the operands that stay in registers (Q, Q': 2 x 64) and the accumulators (O, T:
// 2 x 128) of 32 query rows do not fit one wave next to the score tiles.  Without tangents Q and O
// alone do (64 + 128 in the accumulation file), and that is the first of two passes of the dual
// forward: O and M.  The second pass (TPASS) holds Q, Q' and T (all of the accumulation file), takes
// the final M of the first, so that p = exp2(s - M) needs no running maximum, and writes
// O' = T - mu O and mu.  S is formed twice (seven matrix products instead of six).
//
// Memory side as in fwd_kernel_v2.hpp: direct-to-LDS loads, double buffered, one barrier per tile,
// XOR-swizzled 16-byte chunks, ds_read_b128 for K / K' fragments and the transposing
// ds_read_b64_tr_b16 for V / V'.  A tile is 32 keys (rows are 512 bytes; two stages of 64-key tiles
// would not fit the LDS); a listed 64-key tile is visited as its two halves.
#pragma once
#include <utility>

#include "common.hpp"
#include "mask.hpp"
#include "params.hpp"
#include "pipeline.hpp"

namespace jvpfa {

template <typename T, int D, bool DUAL> struct FwdWideCfg {
  static_assert(sizeof(T) == 2 && D % 32 == 0);
  static constexpr int DV = D;                         // columns of V, V' (all of them)
  static constexpr int NW = 4;
  static constexpr int NT = NW * WAVE;
  static constexpr int BM = NW * 32;
  static constexpr int BN = 32;
  static constexpr int NK = DUAL ? 2 : 1;              // K (, K') and V (, V')
  static constexpr int ROWBK = D * sizeof(T);          // bytes per K-type row (LDS and global)
  static constexpr int ROWBV = DV * sizeof(T);         // bytes per V-type row in LDS (global rows: ROWBK)
  static constexpr int CHK = ROWBK / 16, CHV = ROWBV / 16;
  static constexpr int TILEBK = BN * ROWBK, TILEBV = BN * ROWBV;
  static constexpr int VBASE = NK * TILEBK;            // stage: [K | K' | V | V']
  static constexpr int STAGEB = NK * (TILEBK + TILEBV);
  static constexpr size_t LDS_BYTES = 2 * (size_t)STAGEB;
  static constexpr int IPWK = TILEBK / 1024 / NW;      // direct-load instructions per wave per tile
  static constexpr int IPWV = TILEBV / 1024 / NW;
  static_assert(IPWK >= 1 && IPWV >= 1 && CHK == 32 && CHV == 32);
};

// TPASS (with DUAL): the second pass of the dual forward, see above.
// DROP: dropout on the probabilities (see fwd_kernel.hpp), in both passes.
template <typename T, int D, bool DUAL, int MASK, bool TPASS = false, bool DROP = false>
__global__ __launch_bounds__(256, 1) void fwd_wide_kernel(const FwdParams p) {
  static_assert(!TPASS || DUAL);
  using Cfg = FwdWideCfg<T, D, DUAL>;
  constexpr int DV = Cfg::DV;
  constexpr bool GD = TPASS;  // the accumulation file is full: see mma_vra
  constexpr int BN = Cfg::BN, NK = Cfg::NK;
  constexpr int ROWBK = Cfg::ROWBK, ROWBV = Cfg::ROWBV, TILEBK = Cfg::TILEBK, TILEBV = Cfg::TILEBV;
  constexpr int IPWK = Cfg::IPWK, IPWV = Cfg::IPWV, VBASE = Cfg::VBASE;
  constexpr int KK = D / 16, DB = DV / 32;
  constexpr float NEG_INF = -__builtin_inff();

  extern __shared__ __attribute__((aligned(1024))) unsigned char smem_raw[];
  const uint32_t lds0 = (uint32_t)(uintptr_t)smem_raw;

  const Problem &pr = p.pr;
  const int L = pr.L;
  const int nqb = (L + Cfg::BM - 1) / Cfg::BM;
  const int id = xcd_remap(blockIdx.x, nqb, pr.Z * pr.H);
  const int zh = id / nqb;
  const int rem = id % nqb;
  const int qb = pr.causal ? nqb - 1 - rem : rem;
  const int z = zh / pr.H, h = zh % pr.H;

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid / WAVE), lane = tid % WAVE;
  const int r = lane % 32, g = lane / 32;
  const int pr32 = perm32(r);

  const size_t head = (size_t)zh * L * D;
  const int Lk = pr.Lk;
  const size_t kvhead = ((size_t)z * pr.Hk + h / (pr.H / pr.Hk)) * Lk * D;
  const T *Qg = reinterpret_cast<const T *>(p.q) + head;
  const T *Kg = reinterpret_cast<const T *>(p.k) + kvhead;
  const T *Vg = reinterpret_cast<const T *>(p.v) + kvhead;
  const T *Qtg = DUAL ? reinterpret_cast<const T *>(p.qt) + head : nullptr;
  const T *Ktg = DUAL ? reinterpret_cast<const T *>(p.kt) + kvhead : nullptr;
  const T *Vtg = DUAL ? reinterpret_cast<const T *>(p.vt) + kvhead : nullptr;

  const int q0 = qb * Cfg::BM;
  const int qrow = q0 + wave * 32 + r;
  const int qld = qrow < L ? qrow : L - 1;

  // ---- per-lane constants of the direct loads: instruction i of this wave fills LDS chunks
  // 64*(wave*IPW+i) .. +63 of a tile; this lane's chunk holds (row, logical chunk cp), fetched from
  // the swizzled chunk of the same row in global memory.
  int k_row[IPWK], v_row[IPWV];
  uint32_t k_c[IPWK], v_c[IPWV];
#pragma unroll
  for (int i = 0; i < IPWK; ++i) {
    const int lc = 64 * (wave * IPWK + i) + lane;
    k_row[i] = lc / Cfg::CHK;
    k_c[i] = ((lc % Cfg::CHK) ^ (k_row[i] & 15)) * 16;
  }
#pragma unroll
  for (int i = 0; i < IPWV; ++i) {
    const int lc = 64 * (wave * IPWV + i) + lane;
    v_row[i] = lc / Cfg::CHV;
    v_c[i] = ((lc % Cfg::CHV) ^ swz_v<Cfg::CHV>(v_row[i])) * 16;
  }

  // ---- per-lane LDS read offsets (bytes within a tile)
  // K-type: row perm32(r), logical chunk 2kk + g
  uint32_t koff[KK];
#pragma unroll
  for (int kk = 0; kk < KK; ++kk) koff[kk] = pr32 * ROWBK + (((2 * kk + g) ^ (pr32 & 15)) * 16);
  // V-type (transposing read): lane = 32g + 16a + j addresses key row 8g + 4hh + j/4 (+16c) and the
  // 8-byte half (j>>1)&1 of logical chunk 4db + 2a + (j&1); it receives keys 16c+8g+4hh+(0..3) at
  // column 32db + perm32(16a + j).
  uint32_t voff[DB][2];
  {
    const int a = (lane >> 4) & 1, j = lane & 15;
#pragma unroll
    for (int db = 0; db < DB; ++db) {
#pragma unroll
      for (int hh = 0; hh < 2; ++hh) {
        const int row = 8 * g + 4 * hh + (j >> 2);
        const int ch = (4 * db + 2 * a + (j & 1)) ^ swz_v<Cfg::CHV>(row);
        voff[db][hh] = row * ROWBV + ch * 16 + 8 * ((j >> 1) & 1);
      }
    }
  }

  Frag<T> Qf[KK], Qtf[DUAL ? KK : 1];
#pragma unroll
  for (int kk = 0; kk < KK; ++kk) {
    Qf[kk] = ld8<T>(Qg + (size_t)qld * D + 16 * kk + 8 * g);
    if constexpr (DUAL) Qtf[kk] = ld8<T>(Qtg + (size_t)qld * D + 16 * kk + 8 * g);
  }
#pragma unroll
  for (int kk = 0; kk < KK; ++kk) {
    pin_acc(Qf[kk]);
    if constexpr (DUAL) pin_acc(Qtf[kk]);
  }

  f32x16 Oacc[TPASS ? 1 : DB], Tacc[DUAL ? DB : 1];
#pragma unroll
  for (int db = 0; db < DB; ++db) {
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      if constexpr (!TPASS) Oacc[db][e] = 0.f;
      if constexpr (DUAL) Tacc[db][e] = 0.f;
    }
  }
  float m_i = NEG_INF, l_i = 0.f, mu_i = 0.f;
  // Second pass: S' enters T and mu as S' - c, with c the row's weighted mean of S' over the first tile in which the
  // row has any weight (so tiles skipped because nothing in them is attended do not change it).  O' = T - mu O
  // subtracts two sums of about |S'| |V| whose first one went through 16-bit P S' operands; measured from c both
  // are small wherever one tile holds most of the row's weight (a row with a single key: exactly 0).  p is already
  // normalised by the final M, so c never has to move once it is set.
  float c_i = 0.f;
  if constexpr (TPASS) m_i = qrow < L ? p.M[(size_t)zh * L + qld] : __builtin_inff();  // +inf: a row without keys
  bool c_set = !TPASS || !(m_i < __builtin_inff());  // rows without keys never set c and need none

  const float sl2 = pr.scale * LOG2E;
  const int64_t mrow = MASK != MASK_NONE ? z * pr.ms[0] + h * pr.ms[1] + (int64_t)qld * pr.ms[2] : 0;
  const uint32_t drop_row = DROP ? drop_row_word(pr, zh, qld) : 0u;  // dropout: this lane's query row, see params.hpp
  bool mask_al = false;
  if constexpr (MASK != MASK_NONE) mask_al = mask_rows_aligned<T, MASK>(pr);

  int kend = Lk;
  if constexpr (MASK != MASK_NONE) {
    if (pr.klimit) kend = min(Lk, max(pr.klimit[z], 1));
  }
  if (pr.causal) kend = min(Lk, q0 + Cfg::BM);
  // Tiles visited: the 32-key tiles 0 .. ceil(kend/32)-1, or both halves of every 64-key tile of the
  // caller's list for this query block (ascending; a tile without an attended entry contributes exact
  // zeros, so leaving it out changes nothing).  The second half of the last listed tile is dropped
  // when it lies past the last key.
  const int *tlist = nullptr;
  if constexpr (MASK != MASK_NONE) {
    if (pr.tiles_q) tlist = pr.tiles_q + tile_list_offset_q(pr, z, h, qb);
  }
  const int tmax = (Lk + TILE_W - 1) / TILE_W - 1;  // bounds whatever a list holds
  int ntiles = (kend + BN - 1) / BN;
  if (tlist) {
    const int cnt = min(max(tlist[0], 1), tmax + 1);
    const int last = min(max(tlist[cnt], 0), tmax);
    ntiles = 2 * cnt - (last * TILE_W + BN >= Lk ? 1 : 0);
  }
  // first key of the t-th tile visited, given the list entry that covers it
  auto list_slot = [&](int t) { return tlist ? tlist + 1 + (t >> 1) : reinterpret_cast<const int *>(p.q); };
  auto key_of = [&](int entry, int t) { return tlist ? min(max(entry, 0), tmax) * TILE_W + (t & 1) * BN : t * BN; };

  // The loads of the next tile are issued one instruction at a time, spread over the steps of the
  // current tile's matrix products.  Past the last tile they are pointed at tile 0 again (never
  // read), which keeps every step of the tile loop one straight-line block.
  constexpr int NLOADK = IPWK * NK, NLOAD = NLOADK + IPWV * NK;
  constexpr int NPV = 2 * DB;                  // PV steps: (16-key chunk c, column block db)
  constexpr int NSTEP = KK + NPV;
  int ld_rows = 0;
  uint32_t ld_dst = 0;
  const char *ld_p[4] = {nullptr, nullptr, nullptr, nullptr};  // K, K', V, V'
  auto prepare_loads = [&](int stage, int j0, bool on) {
    j0 = on ? j0 : 0;
    ld_rows = Lk - 1 - j0;  // rows past the end re-read the last row; their scores are masked
    ld_dst = lds0 + stage * Cfg::STAGEB;
    const size_t tb = (size_t)j0 * ROWBK;
    ld_p[0] = reinterpret_cast<const char *>(Kg) + tb;
    ld_p[2] = reinterpret_cast<const char *>(Vg) + tb;
    if constexpr (DUAL) {
      ld_p[1] = reinterpret_cast<const char *>(Ktg) + tb;
      ld_p[3] = reinterpret_cast<const char *>(Vtg) + tb;
    }
  };
  auto load_piece = [&](auto pc) {
    constexpr int pi = decltype(pc)::value;
    if constexpr (pi < NLOADK) {
      constexpr int i = pi / NK, ts = pi % NK;
      const uint32_t off = min(k_row[i], ld_rows) * ROWBK + k_c[i];
      __builtin_amdgcn_global_load_lds((JVPFA_GLB(const void))(ld_p[ts] + off),
                                       (JVPFA_LDS(void))(uintptr_t)(ld_dst + ts * TILEBK + (wave * IPWK + i) * 1024), 16, 0, 0);
    } else {
      constexpr int i = (pi - NLOADK) / NK, ts = (pi - NLOADK) % NK;
      const uint32_t off = min(v_row[i], ld_rows) * ROWBK + v_c[i];
      __builtin_amdgcn_global_load_lds((JVPFA_GLB(const void))(ld_p[2 + ts] + off),
                                       (JVPFA_LDS(void))(uintptr_t)(ld_dst + VBASE + ts * TILEBV + (wave * IPWV + i) * 1024), 16, 0, 0);
    }
  };
  auto load_step = [&](auto gc) {
    constexpr int s = decltype(gc)::value;
    constexpr int lo = (s * NLOAD + NSTEP - 1) / NSTEP, hi = ((s + 1) * NLOAD + NSTEP - 1) / NSTEP;
    static_for<hi - lo>([&](auto dc) { load_piece(std::integral_constant<int, lo + decltype(dc)::value>{}); });
  };

  // One tile: the 32 keys staged at LDS byte address sbase; j0 is the index of its first key.
  // LDS fragment reads run RD-1 steps ahead of the matrix products that consume them; rescaling is
  // lazy (the reference point of the exponentials moves only when a row maximum outgrows it by
  // more than RESCALE_TAU), as in the 64/128 kernel.
  constexpr float RESCALE_TAU = 8.f;
  MaskAhead<T, MASK> mcur[2], mnext[2];  // mask values of this tile and the next: [16-key group]
  const int klim = min(pr.causal ? qrow : 0x7fffffff, Lk - 1);  // keys above this index are masked
  auto tile_body = [&](auto EDGEc, uint32_t sbase, int j0) {
    constexpr bool EDGE = decltype(EDGEc)::value;
    constexpr int NRS = DUAL ? 2 : 1;   // LDS reads per S step
    constexpr int NRV = DUAL ? 4 : 2;   // LDS reads per PV step
    constexpr int RD = 4, PD = RD - 1;
    u32x4 ka[RD], kb[RD];
    auto issue_k = [&](auto kkc) {
      constexpr int kk = decltype(kkc)::value;
      const uint32_t ad = sbase + koff[kk];
      ka[kk % RD] = lds_b128<0>(ad);
      if constexpr (DUAL) kb[kk % RD] = lds_b128<TILEBK>(ad);
    };
    u32x2 va[RD][2], vb[RD][2];
    auto issue_v = [&](auto ic) {
      constexpr int i = decltype(ic)::value, c = i / DB, db = i % DB;
      constexpr int VO = VBASE + c * 16 * ROWBV;
      const uint32_t a0 = sbase + voff[db][0], a1 = sbase + voff[db][1];
      va[i % RD][0] = lds_tr64<VO>(a0);
      va[i % RD][1] = lds_tr64<VO>(a1);
      if constexpr (DUAL) {
        vb[i % RD][0] = lds_tr64<VO + TILEBV>(a0);
        vb[i % RD][1] = lds_tr64<VO + TILEBV>(a1);
      }
    };

    f32x16 S, Sp;
    static_for<PD>([&](auto kkc) { issue_k(kkc); });
    static_for<KK>([&](auto kkc) {
      constexpr int kk = decltype(kkc)::value;
      constexpr int younger = (KK - 1 - kk < PD - 1) ? KK - 1 - kk : PD - 1;
      if constexpr (DUAL) lds_wait<younger * NRS>(ka[kk % RD], kb[kk % RD]);
      else lds_wait<younger * NRS>(ka[kk % RD]);
      if constexpr (kk + PD < KK) issue_k(std::integral_constant<int, kk + PD>{});
      load_step(std::integral_constant<int, kk>{});
      const Frag<T> a = __builtin_bit_cast(Frag<T>, ka[kk % RD]);
      if constexpr (DUAL) mma_vra<kk == 0, GD>(Sp, a, Qtf[kk]);
      mma_vra<kk == 0, GD>(S, a, Qf[kk]);
      if constexpr (DUAL) mma_vra<false, GD>(Sp, __builtin_bit_cast(Frag<T>, kb[kk % RD]), Qf[kk]);
    });
    if constexpr (DUAL) tiles_ready(S, Sp);
    else tiles_ready(S);
    float mx = 0.f;
    constexpr bool general = MASK != MASK_NONE || EDGE;
    if constexpr (general) {
      mx = NEG_INF;
#pragma unroll
      for (int hf = 0; hf < 2; ++hf) {
        const int key0 = j0 + 16 * hf + 8 * g;
        float bias[8];
        bool keep[8];
        if constexpr (MASK != MASK_NONE) {
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            if constexpr (MASK == MASK_ADD) bias[e] = mask_bias_of<T, MASK>(mcur[hf], e);
            if constexpr (MASK == MASK_BOOL) keep[e] = mask_keep_of<T, MASK>(mcur[hf], e);
          }
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          float s = S[8 * hf + e] * sl2;
          if constexpr (MASK == MASK_ADD) s += bias[e];
          if constexpr (MASK == MASK_BOOL) s = keep[e] ? s : NEG_INF;
          if constexpr (EDGE) s = (key0 + e <= klim) ? s : NEG_INF;
          S[8 * hf + e] = s;
          mx = fmaxf(mx, s);
        }
      }
      mx = pair_max(mx);
    } else if constexpr (!TPASS) {
      mx = S[0];
#pragma unroll
      for (int e = 1; e < 16; ++e) mx = fmaxf(mx, S[e]);
      mx = pair_max(mx) * sl2;
    }
    if constexpr (!TPASS) {
      if (__any(mx > m_i + RESCALE_TAU)) {
        const float m_new = fmaxf(m_i, mx);
        const float alpha = fast_exp2(m_i - ((m_new == NEG_INF) ? 0.f : m_new));
        m_i = m_new;
        l_i *= alpha;
        if constexpr (DUAL) mu_i *= alpha;
  #pragma unroll
        for (int db = 0; db < DB; ++db) {
  #pragma unroll
          for (int e = 0; e < 16; ++e) {
            Oacc[db][e] = acc_scale(Oacc[db][e], alpha);
            if constexpr (DUAL) Tacc[db][e] = acc_scale(Tacc[db][e], alpha);
          }
        }
      }
    }
    // V fragments of the first PV steps travel while the softmax runs
    static_for<PD>([&](auto ic) { issue_v(ic); });

    const float m_use = (m_i == NEG_INF) ? 0.f : m_i;
    float rs = 0.f, rmu = 0.f;
    if constexpr (general) {
#pragma unroll
      for (int e = 0; e < 16; ++e) S[e] = fast_exp2(S[e] - m_use);
    } else {
#pragma unroll
      for (int e = 0; e < 16; ++e) S[e] = fast_exp2(__builtin_fmaf(S[e], sl2, -m_use));
    }
    if constexpr (TPASS) {
      if (__any(!c_set)) {  // the first tile or two (a branch among vector instructions only)
        float w0 = 0.f, w1 = 0.f;
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          w0 += S[e];
          w1 = __builtin_fmaf(S[e], Sp[e] * pr.scale, w1);
        }
        w0 += xor32(w0);  // the row's other half of the tile
        w1 += xor32(w1);
        if (!c_set && w0 > 0.f) {
          c_i = w1 / w0;
          c_set = true;
        }
      }
    }
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      rs += S[e];
      if constexpr (DUAL) {
        const float ps = S[e] * __builtin_fmaf(Sp[e], pr.scale, -c_i);
        Sp[e] = ps;
        rmu += ps;
      }
    }
    l_i += rs;
    if constexpr (DUAL) mu_i += rmu;
    if constexpr (DROP) {  // register e holds key j0 + 16(e/8) + 8g + e%8 of this lane's query
      const uint32_t xb = drop_row + (uint32_t)(j0 + 8 * g) * DROP_C_KEY;
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const float ks = drop_scale_of(pr, xb + (uint32_t)(16 * (e / 8) + (e % 8)) * DROP_C_KEY);
        S[e] *= ks;
        if constexpr (DUAL) Sp[e] *= ks;
      }
    }

    Frag<T> pf[2], psf[2];
#pragma unroll
    for (int c = 0; c < 2; ++c) {
      pf[c] = to_frag<T>(S, c);
      if constexpr (DUAL) psf[c] = to_frag<T>(Sp, c);
    }
    static_for<NPV>([&](auto ic) {
      constexpr int i = decltype(ic)::value, c = i / DB, db = i % DB, sl = i % RD;
      constexpr int younger = (NPV - 1 - i < PD - 1) ? NPV - 1 - i : PD - 1;
      if constexpr (DUAL) lds_wait<younger * NRV>(va[sl][0], va[sl][1], vb[sl][0], vb[sl][1]);
      else lds_wait<younger * NRV>(va[sl][0], va[sl][1]);
      if constexpr (i + PD < NPV) issue_v(std::integral_constant<int, i + PD>{});
      load_step(std::integral_constant<int, KK + i>{});
      const u32x4 av = {va[sl][0][0], va[sl][0][1], va[sl][1][0], va[sl][1][1]};
      const Frag<T> a = __builtin_bit_cast(Frag<T>, av);
      if constexpr (!TPASS) mma(Oacc[db], a, pf[c]);
      if constexpr (DUAL) {
        mma(Tacc[db], a, psf[c]);
        const u32x4 bv = {vb[sl][0][0], vb[sl][0][1], vb[sl][1][0], vb[sl][1][1]};
        mma(Tacc[db], __builtin_bit_cast(Frag<T>, bv), pf[c]);
      }
    });
  };

  // mask values of tile t+1 are requested at the top of tile t
  auto fetch_masks = [&](int jn) {
    if constexpr (MASK != MASK_NONE) {
      if (mask_al && jn + BN <= Lk) {
#pragma unroll
        for (int i = 0; i < 2; ++i) mnext[i] = mask_fetch8<T, MASK>(pr, mrow, jn + 16 * i + 8 * g);
      } else {
#pragma unroll
        for (int i = 0; i < 2; ++i) mnext[i] = mask_fetch8_any<T, MASK>(pr, mrow, jn + 16 * i + 8 * g);
      }
    }
  };
  // first keys of the tile of this step and of the next
  int jcur = key_of(tlist ? tlist[1] : 0, 0);
  int jnext = key_of(tlist ? tlist[1 + (min(1, ntiles - 1) >> 1)] : 0, min(1, ntiles - 1));
  fetch_masks(jcur);
  {
    prepare_loads(0, jcur, true);
    static_for<NLOAD>([&](auto pc) { load_piece(pc); });
  }
  auto tile = [&](int t, auto EDGEc) {
    const int stage = t & 1;
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this wave's share of tile t has landed
    __syncthreads();                      // ... everyone's has, and stage^1 is no longer being read
    const int tnext2 = min(t + 2, ntiles - 1);
    int tahead = 0;
    if constexpr (MASK != MASK_NONE) {
      tahead = list_request(list_slot(tnext2));  // read a tile ahead, taken at the end of this one
      mcur[0] = mnext[0];
      mcur[1] = mnext[1];
      fetch_masks(jnext);
    }
    prepare_loads(stage ^ 1, jnext, t + 1 < ntiles);
    tile_body(EDGEc, lds0 + stage * Cfg::STAGEB, jcur);
    int jnext2 = tnext2 * BN;
    if constexpr (MASK != MASK_NONE) jnext2 = key_of(list_take(tahead), tnext2);
    jcur = jnext;
    jnext = jnext2;
  };
  // Tiles that need the general treatment are the last ones; they get a loop of their own so that the
  // common tile carries no limit tests.
  int t_edge = Lk / BN;
  if (pr.causal) t_edge = min(t_edge, q0 / BN);
  if (!(sl2 > 0.f) || (MASK != MASK_NONE && !mask_al)) t_edge = 0;
  int t = 0;
  for (; t < ntiles && jcur < t_edge * BN; ++t) tile(t, std::false_type{});
  for (; t < ntiles; ++t) tile(t, std::true_type{});

  // ---- epilogue ---------------------------------------------------------------------------------
  l_i += xor32(l_i);
  if constexpr (DUAL) mu_i += xor32(mu_i);
  if constexpr (TPASS) {
    // p was normalised by the final M, so T and mu (both measured from c) are final as they stand: T - mu O is the
    // same with or without c, since sum(p) = 1; O comes from the first pass
    if (qrow < L) {
      const T *Og = reinterpret_cast<const T *>(p.o) + head + (size_t)qrow * D;
      T *Otg = reinterpret_cast<T *>(p.ot) + head + (size_t)qrow * D;
#pragma unroll
      for (int db = 0; db < DB; ++db) {
#pragma unroll
        for (int hf = 0; hf < 2; ++hf) {
          const int d0 = 32 * db + 16 * hf + 8 * g;
          const Frag<T> o8 = ld8<T>(Og + d0);
          float t8[8];
#pragma unroll
          for (int e = 0; e < 8; ++e) t8[e] = Tacc[db][8 * hf + e] - mu_i * (float)o8[e];
          store8<T>(Otg + d0, t8);
        }
      }
      if (g == 0) p.mu[(size_t)zh * L + qrow] = __builtin_fmaf(c_i, l_i, mu_i);
    }
  } else {
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
}

}  // namespace jvpfa
