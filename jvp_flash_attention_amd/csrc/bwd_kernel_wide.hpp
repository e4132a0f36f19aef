// dq (PLAIN / DUAL) or dq' (TANGENT) for 16-bit element types with D = 256, on the memory pipeline of
// bwd_kernel_v2.hpp.
//
// The resident operands of 32 query rows (Q, gO, Q', gT: 4 x 64 registers) are the whole
// accumulation file, so, as in fwd_kernel_wide.hpp, two workgroups share a query block: each
// recomputes the score tiles over all of D and accumulates DV = 128 of the dq columns, in ordinary
// vector registers.  Key tiles are 32 rows (K, V, K', V' rows are 512 bytes: two stages of four
// 16 KB tiles fill 128 KB of LDS); a tile is read both ways from its one row-major copy, as there.
#pragma once
#include "bwd_kernel_v2.hpp"

namespace jvpfa {

template <typename T, int D, int DV, int MODE> struct BwdWideCfg {
  static_assert(sizeof(T) == 2 && D == 256 && DV == 128);
  static constexpr int NW = 4;
  static constexpr int NT = NW * WAVE;
  static constexpr int BLK = NW * 32;                 // query rows owned by a workgroup
  static constexpr int BT = 32;                       // keys of a streamed tile
  static constexpr int NS = D / DV;                   // workgroups per query block
  static constexpr int CH = D * sizeof(T) / 16;       // 32 chunks of 16 bytes per row
  static constexpr int ROWB = D * sizeof(T);
  static constexpr int TILEB = BT * ROWB;
  static constexpr int NTILE = MODE == BWD_DUAL ? 4 : 2;
  static constexpr int STAGEB = NTILE * TILEB;
  static constexpr int IPW = TILEB / 1024 / NW;
  static constexpr size_t DQ_LDS = 2 * (size_t)STAGEB;
};

// Chunk swizzle for rows of 512 bytes read both ways: it permutes the low four bits of the chunk
// index.  The row-wise read (16 lanes, 16 rows whose low four bits differ, one logical chunk) needs
// 16 different values; the transposing read (four consecutive rows, an aligned group of four chunks
// each) needs the groups of the four rows apart, i.e. bits 2-3 of the value taken from bits 0-1 of
// the row.
__device__ __forceinline__ int swz_w(int row) { return ((row & 3) << 2) | ((row >> 2) & 3); }

#if defined(__HIP_DEVICE_COMPILE__)
template <typename T, int D, int DV, int MODE, int MASK, bool GO>
__global__ __launch_bounds__(256, 1) void bwdw_dq_kernel(const BwdParams p) {
  using Cfg = BwdWideCfg<T, D, DV, MODE>;
  constexpr bool DUAL = MODE == BWD_DUAL, TAN = MODE == BWD_TANGENT;
  constexpr int CH = Cfg::CH, ROWB = Cfg::ROWB, TILEB = Cfg::TILEB, IPW = Cfg::IPW, BT = Cfg::BT, NS = Cfg::NS;
  constexpr int KK = D / 16, DB = DV / 32;
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem_raw[];
  const uint32_t lds0 = (uint32_t)(uintptr_t)smem_raw;
  const Problem &pr = p.pr;
  const int L = pr.L;
  const int nblk = (L + Cfg::BLK - 1) / Cfg::BLK;
  // the workgroups of one query block follow each other, so they stream the same key tiles from L2
  const int id = xcd_remap(blockIdx.x, nblk * NS, pr.Z * pr.H);
  const int zh = id / (nblk * NS);
  const int rem = id % (nblk * NS);
  const int slice = rem % NS;
  const int qb = pr.causal ? nblk - 1 - rem / NS : rem / NS;
  const int z = zh / pr.H, h = zh % pr.H;
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid / WAVE), lane = tid % WAVE;
  const int r = lane % 32, g = lane / 32, pr32 = perm32(r);
  const size_t head = (size_t)zh * L * D;
  const size_t srow = (size_t)zh * L;
  const int q0 = qb * Cfg::BLK;
  const int qrow = q0 + wave * 32 + r;
  const int qld = qrow < L ? qrow : L - 1;
  constexpr bool has_go = GO;

  // direct loads: instruction i of this wave fills LDS chunks 64*(wave*IPW+i) .. +63 of a tile
  uint32_t ld_o[IPW];
#pragma unroll
  for (int i = 0; i < IPW; ++i) {
    const int lc = 64 * (wave * IPW + i) + lane;
    const int row = lc / CH;
    ld_o[i] = row * ROWB + (((lc % CH) ^ swz_w(row)) * 16);
  }
  uint32_t ld_dst = 0;
  __amdgpu_buffer_rsrc_t ld_rs[4];
  // buffer loads: descriptor = (start of the tile, bytes left in the head); rows past the end of the
  // sequence and tiles that do not exist are out of range and read as zeros
  auto tile_rsrc = [&](const char *base, int j, bool exists) {
    const int rows = exists ? max(pr.Lk - j, 0) : 0;
    return __builtin_amdgcn_make_buffer_rsrc((void *)(base + (size_t)j * ROWB), 0, rows * ROWB, 0x00020000);
  };
  auto load_piece = [&](auto pc) {
    constexpr int pi = decltype(pc)::value, i = pi / Cfg::NTILE, ts = pi % Cfg::NTILE;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(ld_rs[ts], (JVPFA_LDS(void))(uintptr_t)(ld_dst + i * 1024 + ts * TILEB),
                                             16, ld_o[i], 0, 0, 0);
  };
  // row-major fragment: row perm32(r), logical chunk 2kk+g; the swizzle leaves bit 4 of the chunk
  // alone, so steps kk and kk+8 differ by 256 bytes and eight offsets serve all sixteen steps
  uint32_t noff[8];
  {
    const int x = swz_w(pr32);
#pragma unroll
    for (int kk = 0; kk < 8; ++kk) noff[kk] = pr32 * ROWB + (((2 * kk + g) ^ x) * 16);
  }
  // transposed fragment of this workgroup's columns (see fwd_kernel_v2.hpp for the lane pattern)
  uint32_t toff[DB][2];
  {
    const int a_ = (lane >> 4) & 1, j_ = lane & 15;
#pragma unroll
    for (int db = 0; db < DB; ++db) {
#pragma unroll
      for (int hh = 0; hh < 2; ++hh) {
        const int row = 8 * g + 4 * hh + (j_ >> 2);
        const int ch = (4 * db + 2 * a_ + (j_ & 1)) ^ swz_w(row);
        toff[db][hh] = row * ROWB + (16 * slice + ch) * 16 + 8 * ((j_ >> 1) & 1);
      }
    }
  }

  Frag<T> Qf[KK], gOf[TAN ? 1 : KK], Qtf[DUAL ? KK : 1], gTf[(DUAL || TAN) ? KK : 1];
  load_bfrags<KK>(Qf, reinterpret_cast<const T *>(p.q) + head + (size_t)qld * D, g);
  if constexpr (!TAN) {
    if constexpr (has_go) load_bfrags<KK>(gOf, reinterpret_cast<const T *>(p.go) + head + (size_t)qld * D, g);
  }
  if constexpr (DUAL) load_bfrags<KK>(Qtf, reinterpret_cast<const T *>(p.qt) + head + (size_t)qld * D, g);
  if constexpr (DUAL || TAN) load_bfrags<KK>(gTf, reinterpret_cast<const T *>(p.gt) + head + (size_t)qld * D, g);
#pragma unroll
  for (int kk = 0; kk < KK; ++kk) {
    pin_acc(Qf[kk]);
    if constexpr (!TAN && has_go) pin_acc(gOf[kk]);
    if constexpr (DUAL) pin_acc(Qtf[kk]);
    if constexpr (DUAL || TAN) pin_acc(gTf[kk]);
  }

  const float Mq = qrow < L ? p.M[srow + qld] : __builtin_inff();
  const float d1 = (MODE == BWD_PLAIN) ? p.d1[srow + qld] : 0.f;
  const float mu = DUAL ? p.mu[srow + qld] : 0.f;
  const float av = (DUAL || TAN) ? p.a[srow + qld] : 0.f;
  const float dsum = DUAL ? p.d2[srow + qld] : 0.f;

  f32x16 acc[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db) zero_acc(acc[db]);

  const float sl2 = pr.scale * LOG2E;
  const int64_t mrow = MASK != MASK_NONE ? z * pr.ms[0] + h * pr.ms[1] + (int64_t)qld * pr.ms[2] : 0;
  bool mask_al = false;
  if constexpr (MASK != MASK_NONE) mask_al = mask_rows_aligned<T, MASK>(pr);
  const int Lk = pr.Lk;
  const size_t kvhead = ((size_t)z * pr.Hk + h / (pr.H / pr.Hk)) * Lk * D;
  const char *Kb = reinterpret_cast<const char *>(p.k) + kvhead * sizeof(T);
  const char *Vb = reinterpret_cast<const char *>(p.v) + kvhead * sizeof(T);
  const char *Ktb = DUAL ? reinterpret_cast<const char *>(p.kt) + kvhead * sizeof(T) : nullptr;
  const char *Vtb = DUAL ? reinterpret_cast<const char *>(p.vt) + kvhead * sizeof(T) : nullptr;

  int kend = pr.causal ? min(Lk, q0 + Cfg::BLK) : Lk;
  if constexpr (MASK != MASK_NONE) {
    if (pr.klimit) kend = min(kend, max(pr.klimit[z], 1));
  }
  const int ntiles = (kend + BT - 1) / BT;
  // tile slots in a stage: 0 K, 1 V, 2 K', 3 V'
  constexpr int NLOAD = IPW * Cfg::NTILE;
  constexpr int NACC = DUAL ? 2 : 1;
  constexpr int NPV = 2 * (DB / 2);  // accumulation steps: (16-key chunk c, pair of d-blocks)
  constexpr int NSTEP = KK + NPV;
  auto prepare_loads = [&](int stage, int j0, bool on) {
    ld_dst = lds0 + stage * Cfg::STAGEB + (wave * IPW) * 1024;
    ld_rs[0] = tile_rsrc(Kb, j0, on);
    ld_rs[1] = tile_rsrc(Vb, j0, on);
    if constexpr (DUAL) {
      ld_rs[2] = tile_rsrc(Ktb, j0, on);
      ld_rs[3] = tile_rsrc(Vtb, j0, on);
    }
  };
  auto load_step = [&](auto gc) {
    constexpr int gi = decltype(gc)::value;
    constexpr int NSPREAD = JVPFA_BWD_SPREAD(NSTEP);
    if constexpr (gi < NSPREAD) {
      constexpr int lo = (gi * NLOAD + NSPREAD - 1) / NSPREAD, hi = ((gi + 1) * NLOAD + NSPREAD - 1) / NSPREAD;
      static_for<hi - lo>([&](auto dc) { load_piece(std::integral_constant<int, lo + decltype(dc)::value>{}); });
    }
  };

  MaskAhead<T, MASK> mcur[2], mnext[2];  // mask values of this tile and the next: [16-key group]
  const int klim = min(pr.causal ? qrow : 0x7fffffff, Lk - 1);  // keys above this index are masked
  // EDGE: the tile may cross the causal diagonal or the end of the sequence
  auto tile_body = [&](auto EDGEc, uint32_t sbase, int j0) {
    constexpr bool EDGE = decltype(EDGEc)::value;
    // ---- recompute: S, (S', dP, A, B) ----------------------------------------------------------
    FragN fk[2], fv[2], fkt[2], fvt[2];
    auto issue_n = [&](auto kkc) {
      constexpr int kk = decltype(kkc)::value, sl = kk % 2, HI = (kk / 8) * 256;
      const uint32_t ad = sbase + noff[kk % 8];
      fk[sl].v = lds_b128<HI>(ad);
      fv[sl].v = lds_b128<HI + TILEB>(ad);
      if constexpr (DUAL) {
        fkt[sl].v = lds_b128<HI + 2 * TILEB>(ad);
        fvt[sl].v = lds_b128<HI + 3 * TILEB>(ad);
      }
    };
    constexpr int NRN = DUAL ? 4 : 2;
    constexpr bool GD = DUAL;  // the accumulation file is full: see mma_vra
    f32x16 S, dP, Sp, At;  // DUAL: dP also collects V' gT^T (the B term)
    issue_n(std::integral_constant<int, 0>{});
    static_for<KK>([&](auto kkc) {
      constexpr int kk = decltype(kkc)::value, sl = kk % 2;
      constexpr bool F = kk == 0;
      if constexpr (kk + 1 < KK) issue_n(std::integral_constant<int, kk + 1>{});
      if constexpr (DUAL) lds_wait<(kk + 1 < KK) ? NRN : 0>(fk[sl], fv[sl], fkt[sl], fvt[sl]);
      else lds_wait<(kk + 1 < KK) ? NRN : 0>(fk[sl], fv[sl]);
      load_step(std::integral_constant<int, kk>{});
      const Frag<T> k_ = as_frag<T>(fk[sl]), v_ = as_frag<T>(fv[sl]);
      mma_vra<F, GD>(S, k_, Qf[kk]);
      if constexpr (MODE == BWD_PLAIN) mma_vra<F, GD>(dP, v_, gOf[kk]);
      if constexpr (TAN) mma_vra<F, GD>(At, v_, gTf[kk]);
      if constexpr (DUAL) {
        if constexpr (has_go) mma_vra<F, GD>(dP, v_, gOf[kk]);
        mma_vra<F, GD>(Sp, k_, Qtf[kk]);
        mma_vra<F, GD>(At, v_, gTf[kk]);
        mma_vra<false, GD>(Sp, as_frag<T>(fkt[sl]), Qf[kk]);
        mma_vra<F && !has_go, GD>(dP, as_frag<T>(fvt[sl]), gTf[kk]);
      }
    });
    if constexpr (DUAL) tiles_ready(S, dP, Sp, At);
    else if constexpr (TAN) tiles_ready(S, At);
    else tiles_ready(S, dP);

    // ---- P and the score gradients -------------------------------------------------------------
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
        const int i = 8 * hf + e;
        float s = S[i] * sl2;
        if constexpr (MASK == MASK_ADD) s += bias[e];
        float pv = fast_exp2(s - Mq);
        if constexpr (MASK == MASK_BOOL) pv = keep[e] ? pv : 0.f;
        if constexpr (EDGE) pv = (key0 + e <= klim) ? pv : 0.f;
        if constexpr (MODE == BWD_PLAIN) {
          S[i] = pv * (dP[i] - d1);
        } else if constexpr (DUAL) {
          const float sp = Sp[i] * pr.scale, am = At[i] - av;
          Sp[i] = pv * am;
          S[i] = pv * (dP[i] + am * sp - At[i] * mu - dsum);
        } else {
          S[i] = pv * (At[i] - av);
        }
      }
    }
    Frag<T> dsf[2], dspf[2];
#pragma unroll
    for (int c = 0; c < 2; ++c) {
      dsf[c] = to_frag<T>(S, c);
      if constexpr (DUAL) dspf[c] = to_frag<T>(Sp, c);
    }

    // ---- dQ^T += K^T dS^T (+ K'^T dS'^T) on this workgroup's columns -----------------------------
    FragT tk[2][2], tkt[2][2];  // [ring slot][d-block of the pair]
    auto issue_t = [&](auto ic) {
      constexpr int i = decltype(ic)::value, c = i / (DB / 2), dp = i % (DB / 2), sl = i % 2;
      constexpr int TO = c * 16 * ROWB;
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const uint32_t a0 = sbase + toff[2 * dp + u][0], a1 = sbase + toff[2 * dp + u][1];
        tk[sl][u].lo = lds_tr64<TO>(a0);
        tk[sl][u].hi = lds_tr64<TO>(a1);
        if constexpr (DUAL) {
          tkt[sl][u].lo = lds_tr64<TO + 2 * TILEB>(a0);
          tkt[sl][u].hi = lds_tr64<TO + 2 * TILEB>(a1);
        }
      }
    };
    constexpr int NRT = 4 * NACC;
    issue_t(std::integral_constant<int, 0>{});
    static_for<NPV>([&](auto ic) {
      constexpr int i = decltype(ic)::value, c = i / (DB / 2), dp = i % (DB / 2), sl = i % 2;
      if constexpr (i + 1 < NPV) issue_t(std::integral_constant<int, i + 1>{});
      if constexpr (DUAL) lds_wait<(i + 1 < NPV) ? NRT : 0>(tk[sl][0], tk[sl][1], tkt[sl][0], tkt[sl][1]);
      else lds_wait<(i + 1 < NPV) ? NRT : 0>(tk[sl][0], tk[sl][1]);
      load_step(std::integral_constant<int, KK + i>{});
      mma(acc[2 * dp], as_frag<T>(tk[sl][0]), dsf[c]);
      mma(acc[2 * dp + 1], as_frag<T>(tk[sl][1]), dsf[c]);
      if constexpr (DUAL) {
        mma(acc[2 * dp], as_frag<T>(tkt[sl][0]), dspf[c]);
        mma(acc[2 * dp + 1], as_frag<T>(tkt[sl][1]), dspf[c]);
      }
    });
  };

  // mask values of tile t+1 are requested at the top of tile t
  auto fetch_masks = [&](int tn) {
    if constexpr (MASK != MASK_NONE) {
      const int jn = tn * BT;
      if (mask_al && jn + BT <= Lk) {
#pragma unroll
        for (int i = 0; i < 2; ++i) mnext[i] = mask_fetch8<T, MASK>(pr, mrow, jn + 16 * i + 8 * g);
      } else {
#pragma unroll
        for (int i = 0; i < 2; ++i) mnext[i] = mask_fetch8_any<T, MASK>(pr, mrow, jn + 16 * i + 8 * g);
      }
    }
  };
  fetch_masks(0);
  prepare_loads(0, 0, true);
  static_for<NLOAD>([&](auto pc) { load_piece(pc); });
  auto tile = [&](int t, auto EDGEc) {
    const int stage = t & 1;
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this wave's share of tile t has landed
    __syncthreads();                      // ... everyone's has, and stage^1 is no longer being read
    if constexpr (MASK != MASK_NONE) {
      mcur[0] = mnext[0];
      mcur[1] = mnext[1];
      fetch_masks(min(t + 1, ntiles - 1));
    }
    prepare_loads(stage ^ 1, (t + 1) * BT, t + 1 < ntiles);
    tile_body(EDGEc, lds0 + stage * Cfg::STAGEB, t * BT);
  };
  // tiles that cross the diagonal or the end of the sequence are the last ones
  int t_edge = Lk / BT;
  if (pr.causal) t_edge = min(t_edge, q0 / BT);
  if (MASK != MASK_NONE && !mask_al) t_edge = 0;
  int t = 0;
  for (; t < ntiles && t < t_edge; ++t) tile(t, std::false_type{});
  for (; t < ntiles; ++t) tile(t, std::true_type{});
  __builtin_amdgcn_s_waitcnt(0x0F70);  // the redirected loads of the last iteration must not outlive the kernel

  if (qrow < L) {
    T *out = reinterpret_cast<T *>(TAN ? p.dqt : p.dq) + head + (size_t)qrow * D + slice * DV;
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
#else
template <typename T, int D, int DV, int MODE, int MASK, bool GO>
__global__ __launch_bounds__(256, 1) void bwdw_dq_kernel(const BwdParams p) {}
#endif

}  // namespace jvpfa
