// Backward kernels for 16-bit element types (bf16 / fp16), D in {32, 64, 128}, on the forward's memory
// pipeline: 64-row tiles of the streamed tensors go global -> LDS with direct-to-LDS loads, double
// buffered and issued one instruction at a time between the matrix products of the current tile;
// tiles stay row-major (XOR-swizzled 16-byte chunks) and are read both ways from that one copy:
// ds_read_b128 gives the operand of the recomputed products (contraction over d), the transposing
// ds_read_b64_tr_b16 gives the operand of the gradient accumulations (contraction over the
// streamed index).  LDS reads are issued one step ahead of their matrix products.
//
// Mathematics, modes and the reference lines it replaces: see bwd_kernel.hpp.  In BWD_DUAL the
// pre-pass statistic d2 already contains d1 (d2 := d1 + rowsum(gT*O') - a*mu).
#pragma once
#include "common.hpp"
#include "mask.hpp"
#include "params.hpp"
#include "pipeline.hpp"

namespace jvpfa {

template <typename T, int D, int MODE> struct Bwd2Cfg {
  static constexpr int NW = 4;
  static constexpr int NT = NW * WAVE;
  static constexpr int BLK = NW * 32;                 // rows owned by a workgroup
  static constexpr int BT = 64;                       // rows of a streamed tile
  static constexpr int CH = D * sizeof(T) / 16;
  static constexpr int ROWB = D * sizeof(T);
  static constexpr int TILEB = BT * ROWB;
  static constexpr int NTILE = MODE == BWD_DUAL ? 4 : 2;
  static constexpr int STAGEB = NTILE * TILEB;
  static constexpr int IPW = TILEB / 1024 / NW;
  static constexpr int NSTAT = MODE == BWD_DUAL ? 4 : 2;
  static constexpr int STATB = NSTAT * BT * 4;        // row statistics of a query tile (dk/dv only)
  static constexpr size_t DQ_LDS = 2 * (size_t)STAGEB;
  static constexpr size_t DKV_LDS = 2 * (size_t)STAGEB + 2 * (size_t)STATB;
  // MASK_TILE: two stages of a 64-query x 128-key tile of a 16-bit additive mask behind the statistics; where
  // two do not fit (the dual mode at D = 128) one, which every wave empties into registers at the top of a tile,
  // in front of a second barrier, before the direct loads of the tile refill it
  static constexpr int MTILEB = BT * 256;
  static constexpr bool MTILE_SINGLE = DKV_LDS + 2 * (size_t)MTILEB > 160 * 1024;
  static constexpr size_t DKV_LDS_MTILE = DKV_LDS + (MTILE_SINGLE ? 1 : 2) * (size_t)MTILEB;
};

// One LDS fragment (8 elements per lane) read ahead with lds_b128 / two lds_tr64.
struct FragN { u32x4 v; };
struct FragT { u32x2 lo, hi; };
template <typename T> __device__ __forceinline__ Frag<T> as_frag(const FragN &f) { return __builtin_bit_cast(Frag<T>, f.v); }
template <typename T> __device__ __forceinline__ Frag<T> as_frag(const FragT &f) {
  const u32x4 v = {f.lo[0], f.lo[1], f.hi[0], f.hi[1]};
  return __builtin_bit_cast(Frag<T>, v);
}
template <int N> __device__ __forceinline__ void lds_wait(FragN &a, FragN &b) { lds_wait<N>(a.v, b.v); }
template <int N> __device__ __forceinline__ void lds_wait(FragN &a, FragN &b, FragN &c, FragN &d) {
  asm volatile("s_waitcnt lgkmcnt(%4)" : "+v"(a.v), "+v"(b.v), "+v"(c.v), "+v"(d.v) : "n"(N));
}
template <int N> __device__ __forceinline__ void lds_wait(FragT &a, FragT &b) { lds_wait<N>(a.lo, a.hi, b.lo, b.hi); }
template <int N> __device__ __forceinline__ void lds_wait(FragT &a, FragT &b, FragT &c, FragT &d) {
  asm volatile("s_waitcnt lgkmcnt(%8)"
               : "+v"(a.lo), "+v"(a.hi), "+v"(b.lo), "+v"(b.hi), "+v"(c.lo), "+v"(c.hi), "+v"(d.lo), "+v"(d.hi)
               : "n"(N));
}
template <int N> __device__ __forceinline__ void lds_wait4(u32x4 &a, u32x4 &b, u32x4 &c, u32x4 &d) {
  asm volatile("s_waitcnt lgkmcnt(%4)" : "+v"(a), "+v"(b), "+v"(c), "+v"(d) : "n"(N));
}

// Everything the two kernels share: tile geometry, direct loads spread over steps, fragment reads.
// SLOTn are LDS tile slots inside a stage; a tile is BT rows, row-major, chunks swizzled by swz_u.
// the loads of the next tile are spread over the first three quarters of a tile's steps
constexpr int bwd_spread(int nstep) { return 3 * nstep / 4; }
#define JVPFA_BWD2_COMMON(Cfg, STREAMED_ROWS, OWN_ROWS, OWN_HEADS)                                                                                      \
  constexpr int CH = Cfg::CH, ROWB = Cfg::ROWB, TILEB = Cfg::TILEB, IPW = Cfg::IPW, BT = Cfg::BT;                   \
  constexpr int KK = D / 16, DB = D / 32;                                                                           \
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem_raw[];                                        \
  const uint32_t lds0 = (uint32_t)(uintptr_t)smem_raw;                                                              \
  const Problem &pr = p.pr;                                                                                         \
  const int L = pr.L;                                                                                               \
  /* a workgroup owns 128 of the OWN_ROWS rows of one (z, head out of OWN_HEADS) */                               \
  const int nblk = ((OWN_ROWS) + Cfg::BLK - 1) / Cfg::BLK;                                                          \
  const int id = xcd_remap(bid, nblk, pr.Z * (OWN_HEADS));                                                   \
  const int zh = id / nblk;                                                                                         \
  const int z = zh / (OWN_HEADS), h = zh % (OWN_HEADS);                                                             \
  const int tid = threadIdx.x;                                                                                      \
  const int wave = __builtin_amdgcn_readfirstlane(tid / WAVE), lane = tid % WAVE;                                   \
  const int r = lane % 32, g = lane / 32, pr32 = perm32(r);                                                         \
  const size_t head = (size_t)zh * (OWN_ROWS) * D;                                                                  \
  const size_t srow = (size_t)zh * (OWN_ROWS);                                                                      \
  (void)z; (void)h; (void)srow;                                                                                     \
  /* direct loads: instruction i of this wave fills LDS chunks 64*(wave*IPW+i) .. +63 of a tile */                   \
  int ld_row[IPW];                                                                                                  \
  uint32_t ld_c[IPW];                                                                                               \
  _Pragma("unroll") for (int i = 0; i < IPW; ++i) {                                                                 \
    const int lc = 64 * (wave * IPW + i) + lane;                                                                    \
    ld_row[i] = lc / CH;                                                                                            \
    ld_c[i] = ((lc % CH) ^ swz_u<CH>(lc / CH)) * 16;                                                                \
  }                                                                                                                 \
  /* buffer loads: descriptor = (start of the tile, bytes left in the head), per-lane offset constant; rows */      \
  /* past the end of the sequence and tiles that do not exist are out of range and read as zeros */                \
  uint32_t ld_o[IPW];                                                                                               \
  _Pragma("unroll") for (int i = 0; i < IPW; ++i) ld_o[i] = ld_row[i] * ROWB + ld_c[i];                            \
  uint32_t ld_dst = 0;                                                                                              \
  __amdgpu_buffer_rsrc_t ld_rs[4];                                                                                  \
  auto tile_rsrc = [&](const char *base, int j, bool exists) {                                                      \
    const int rows = exists ? max((STREAMED_ROWS) - j, 0) : 0;                                                                    \
    return __builtin_amdgcn_make_buffer_rsrc((void *)(base + (size_t)j * ROWB), 0, rows * ROWB, 0x00020000);       \
  };                                                                                                                \
  auto load_piece = [&](auto pc) {                                                                                  \
    constexpr int pi = decltype(pc)::value, i = pi / Cfg::NTILE, ts = pi % Cfg::NTILE;                              \
    __builtin_amdgcn_raw_ptr_buffer_load_lds(ld_rs[ts], (JVPFA_LDS(void))(uintptr_t)(ld_dst + i * 1024 + ts * TILEB),  \
                                             16, ld_o[i], 0, 0, 0);                                                 \
  };                                                                                                                \
  /* row-major fragment (rows = streamed index, contraction over d): row 32hb + perm32(r), chunk 2kk+g */           \
  uint32_t noff[KK];                                                                                                \
  {                                                                                                                 \
    const int x = swz_u<CH>(pr32);                                                                                  \
    _Pragma("unroll") for (int kk = 0; kk < KK; ++kk) noff[kk] = pr32 * ROWB + (((2 * kk + g) ^ x) * 16);           \
  }                                                                                                                 \
  /* transposed fragment (rows = d, contraction over the streamed index), see fwd_kernel_v2.hpp */                  \
  uint32_t toff[DB][2];                                                                                             \
  {                                                                                                                 \
    const int a_ = (lane >> 4) & 1, j_ = lane & 15;                                                                 \
    _Pragma("unroll") for (int db = 0; db < DB; ++db) {                                                             \
      _Pragma("unroll") for (int hh = 0; hh < 2; ++hh) {                                                            \
        const int row = 8 * g + 4 * hh + (j_ >> 2);                                                                 \
        const int ch = (4 * db + 2 * a_ + (j_ & 1)) ^ swz_u<CH>(row);                                               \
        toff[db][hh] = row * ROWB + ch * 16 + 8 * ((j_ >> 1) & 1);                                                  \
      }                                                                                                             \
    }                                                                                                               \
  }

template <int KK, typename T>
__device__ __forceinline__ void load_bfrags(Frag<T> *f, const T *row, int g) {
#pragma unroll
  for (int kk = 0; kk < KK; ++kk) f[kk] = ld8<T>(row + 16 * kk + 8 * g);
}

__device__ __forceinline__ void zero_acc(f32x16 &x) {
#pragma unroll
  for (int e = 0; e < 16; ++e) x[e] = 0.f;
}

// ------------------------------------------------------------------------------------------------
// dq (PLAIN / DUAL) or dq' (TANGENT): workgroup = 128 query rows, loop over 64-key tiles of
// K, V (, K', V').  Scores are transposed (lane = query) so dS is the B operand of dQ^T += K^T dS^T.
#if defined(__HIP_DEVICE_COMPILE__)  // the host pass only needs the launch stubs (and has no buffer descriptor type)
// SIX (dual mode only): dq' = scale dS' K as well, from the K fragments and the dS' tiles that dq already has.
// DROP: dropout (see bwd_kernel.hpp): gO V^T, gT V^T and gT V'^T reach the logits through the kept, rescaled
// entries only.
// LEAN: one tile loop (every tile takes the limit tests) instead of an interior loop and an edge loop: less for
// the compiler to keep in registers, for the variant that must stay within 256 of them.
template <typename T, int D, int MODE, int MASK, bool GO, bool SIX, bool DROP = false, bool LEAN = false>
__device__ __forceinline__ void bwd2_dq_body(const BwdParams &p, const int bid) {
  using Cfg = Bwd2Cfg<T, D, MODE>;
  constexpr bool DUAL = MODE == BWD_DUAL, TAN = MODE == BWD_TANGENT;
  static_assert(!SIX || DUAL, "dq' rides on the dual mode");
  JVPFA_BWD2_COMMON(Cfg, pr.Lk, pr.L, pr.H)  // owns query rows, streams key tiles
  const int qb = pr.causal ? nblk - 1 - id % nblk : id % nblk;
  const int q0 = qb * Cfg::BLK;
  const int qrow = q0 + wave * 32 + r;
  const int qld = qrow < L ? qrow : L - 1;
  constexpr bool has_go = GO;  // compile-time: a run-time test here would split every step into its own block

  Frag<T> Qf[KK], gOf[TAN ? 1 : KK], Qtf[DUAL ? KK : 1], gTf[(DUAL || TAN) ? KK : 1];
  load_bfrags<KK>(Qf, reinterpret_cast<const T *>(p.q) + head + (size_t)qld * D, g);
  if constexpr (!TAN) {
    if constexpr (has_go) load_bfrags<KK>(gOf, reinterpret_cast<const T *>(p.go) + head + (size_t)qld * D, g);
  }
  if constexpr (DUAL) load_bfrags<KK>(Qtf, reinterpret_cast<const T *>(p.qt) + head + (size_t)qld * D, g);
  if constexpr (DUAL || TAN) load_bfrags<KK>(gTf, reinterpret_cast<const T *>(p.gt) + head + (size_t)qld * D, g);
  // the resident operands live in the accumulation register file from here on (with dq' at D = 128 that
  // file is full with the two accumulators and three of them: gO stays in vector registers)
  constexpr bool GO_V = SIX && D == 128;
#pragma unroll
  for (int kk = 0; kk < KK; ++kk) {
    pin_acc(Qf[kk]);
    if constexpr (!TAN && has_go && !GO_V) pin_acc(gOf[kk]);
    if constexpr (DUAL) pin_acc(Qtf[kk]);
    if constexpr (DUAL || TAN) pin_acc(gTf[kk]);
  }

  const float Mq = qrow < L ? p.M[srow + qld] : __builtin_inff();
  const uint32_t drop_row = DROP ? drop_row_word(pr, zh, qld) : 0u;  // dropout: this lane's query row
  const float d1 = (MODE == BWD_PLAIN) ? p.d1[srow + qld] : 0.f;
  const float mu = DUAL ? p.mu[srow + qld] : 0.f;
  const float av = (DUAL || TAN) ? p.a[srow + qld] : 0.f;
  const float dsum = DUAL ? p.d2[srow + qld] : 0.f;

  f32x16 acc[DB], accT[SIX ? DB : 1];
#pragma unroll
  for (int db = 0; db < DB; ++db) {
    zero_acc(acc[db]);
    if constexpr (SIX) zero_acc(accT[db]);
  }

  const float sl2 = pr.scale * LOG2E;
  const int64_t mrow = MASK != MASK_NONE ? z * pr.ms[0] + h * pr.ms[1] + (int64_t)qld * pr.ms[2] : 0;
  bool mask_al = false;  // mask rows can be fetched with aligned vector loads
  if constexpr (MASK != MASK_NONE) mask_al = mask_rows_aligned<T, MASK>(pr);
  // keys: Lk of them, in head h / (H / Hk) of the key/value tensors (L and h themselves for the
  // shapes the reference admits)
  const int Lk = pr.Lk;
  const size_t kvhead = ((size_t)z * pr.Hk + h / (pr.H / pr.Hk)) * Lk * D;
  const char *Kb = reinterpret_cast<const char *>(p.k) + kvhead * sizeof(T);
  const char *Vb = reinterpret_cast<const char *>(p.v) + kvhead * sizeof(T);
  const char *Ktb = DUAL ? reinterpret_cast<const char *>(p.kt) + kvhead * sizeof(T) : nullptr;
  const char *Vtb = DUAL ? reinterpret_cast<const char *>(p.vt) + kvhead * sizeof(T) : nullptr;

  int kend = pr.causal ? min(Lk, q0 + Cfg::BLK) : Lk;
  if constexpr (MASK != MASK_NONE) {  // key tiles that the caller's hint declares fully masked are not visited
    if (pr.klimit) kend = min(kend, max(pr.klimit[z], 1));
  }
  // Key tiles visited: 0 .. ceil(kend/BT)-1, or the caller's list of the tiles of this query block
  // that hold an attended entry (ascending); tile_at(i) is the i-th one.
  const int *tlist = nullptr;
  if constexpr (MASK != MASK_NONE) {
    if (pr.tiles_q) tlist = pr.tiles_q + tile_list_offset_q(pr, z, h, qb);
  }
  const int tmax = (Lk + BT - 1) / BT - 1;  // index of the last tile of the sequence: bounds whatever a list holds
  const int ntiles = tlist ? min(max(tlist[0], 1), tmax + 1) : (kend + BT - 1) / BT;
  // List elements are requested a tile ahead, unconditionally (from a harmless address when there is
  // no list: a branch around the read would split the tile loop's straight-line body).
  auto list_slot = [&](int i) { return tlist ? tlist + 1 + i : reinterpret_cast<const int *>(p.q); };
  // tile slots in a stage: 0 K, 1 V, 2 K', 3 V'
  constexpr int NLOAD = IPW * Cfg::NTILE;
  constexpr int NACC = DUAL ? 2 : 1;            // operand tensors of the accumulation (K, K')
  constexpr int PW = DB >= 2 ? 2 : 1;           // d-blocks per accumulation step (one for D = 32)
  constexpr int NDP = DB / PW;
  constexpr int NPV = 2 * NDP;                  // accumulation steps of a half: (chunk c, group of PW d-blocks)
  constexpr int NSTEP = 2 * (KK + NPV);
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
    // spread over the first NSPREAD steps only: the last load then has time to land before the barrier
    constexpr int NSPREAD = bwd_spread(NSTEP);
    if constexpr (gi < NSPREAD) {
      constexpr int lo = (gi * NLOAD + NSPREAD - 1) / NSPREAD, hi = ((gi + 1) * NLOAD + NSPREAD - 1) / NSPREAD;
      static_for<hi - lo>([&](auto dc) { load_piece(std::integral_constant<int, lo + decltype(dc)::value>{}); });
    }
  };

  MaskAhead<T, MASK> mcur[2][2], mnext[2][2];  // mask values of this tile and the next: [half tile][16-key group]
  // EDGE: the half tile may cross the causal diagonal or the end of the sequence
  auto half_tile = [&](auto HBc, auto EDGEc, uint32_t sbase, int jh) {
    constexpr int HB = decltype(HBc)::value;
    constexpr bool EDGE = decltype(EDGEc)::value;
    constexpr int RO = HB * 32 * ROWB;
    // ---- recompute: S, (S', dP, A, B) --------------------------------------------------------
    FragN fk[2], fv[2], fkt[2], fvt[2];
    auto issue_n = [&](auto kkc) {
      constexpr int kk = decltype(kkc)::value, sl = kk % 2;
      const uint32_t ad = sbase + noff[kk];
      fk[sl].v = lds_b128<RO>(ad);
      fv[sl].v = lds_b128<RO + TILEB>(ad);
      if constexpr (DUAL) {
        fkt[sl].v = lds_b128<RO + 2 * TILEB>(ad);
        fvt[sl].v = lds_b128<RO + 3 * TILEB>(ad);
      }
    };
    constexpr int NRN = DUAL ? 4 : 2;
    // mask values of this half tile: requested a whole tile earlier (see tile() below)
    MaskAhead<T, MASK> mah[2];
    if constexpr (MASK != MASK_NONE) {
      mah[0] = mcur[HB][0];
      mah[1] = mcur[HB][1];
    }
    // tiles in ordinary vector registers; in DUAL, dP also collects V' gT^T (the B term)
    f32x16 S, dP, Sp, At;
    issue_n(std::integral_constant<int, 0>{});
    static_for<KK>([&](auto kkc) {
      constexpr int kk = decltype(kkc)::value, sl = kk % 2;
      constexpr bool F = kk == 0;
      if constexpr (kk + 1 < KK) issue_n(std::integral_constant<int, kk + 1>{});
      if constexpr (DUAL) lds_wait<(kk + 1 < KK) ? NRN : 0>(fk[sl], fv[sl], fkt[sl], fvt[sl]);
      else lds_wait<(kk + 1 < KK) ? NRN : 0>(fk[sl], fv[sl]);
      load_step(std::integral_constant<int, HB * KK + kk>{});
      const Frag<T> k_ = as_frag<T>(fk[sl]), v_ = as_frag<T>(fv[sl]);
      mma_vra<F>(S, k_, Qf[kk]);
      if constexpr (MODE == BWD_PLAIN) mma_vra<F>(dP, v_, gOf[kk]);
      if constexpr (TAN) mma_vra<F>(At, v_, gTf[kk]);
      if constexpr (DUAL) {
        if constexpr (has_go && GO_V) mma_vrv<F>(dP, v_, gOf[kk]);
        else if constexpr (has_go) mma_vra<F>(dP, v_, gOf[kk]);
        mma_vra<F>(Sp, k_, Qtf[kk]);
        mma_vra<F>(At, v_, gTf[kk]);
        mma_vra<false>(Sp, as_frag<T>(fkt[sl]), Qf[kk]);
        mma_vra<F && !has_go>(dP, as_frag<T>(fvt[sl]), gTf[kk]);
      }
    });
    if constexpr (DUAL) tiles_ready(S, dP, Sp, At);
    else if constexpr (TAN) tiles_ready(S, At);
    else tiles_ready(S, dP);

    // ---- P and the score gradients -------------------------------------------------------------
    const int klim = min(pr.causal ? qrow : 0x7fffffff, Lk - 1);  // keys above this index are masked
#pragma unroll
    for (int hf = 0; hf < 2; ++hf) {
      const int key0 = jh + 16 * hf + 8 * g;
      float bias[8];
      bool keep[8];
      if constexpr (MASK != MASK_NONE) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          // the mask value and the row's reference point in one term: the exponent is then one fused multiply-add
          if constexpr (MASK == MASK_ADD) bias[e] = fmaf((float)mah[hf].f[e], LOG2E, -Mq);
          if constexpr (MASK == MASK_BOOL) keep[e] = mask_keep_of<T, MASK>(mah[hf], e);
        }
      }
      const uint32_t xb = DROP ? drop_row + (uint32_t)key0 * DROP_C_KEY : 0u;  // dropout word of key key0, see params.hpp
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int i = 8 * hf + e;
        float pv;
        if constexpr (MASK == MASK_ADD) pv = fast_exp2(fmaf(S[i], sl2, bias[e]));
        else pv = fast_exp2(S[i] * sl2 - Mq);
        if constexpr (MASK == MASK_BOOL) pv = keep[e] ? pv : 0.f;
        if constexpr (EDGE) pv = (key0 + e <= klim) ? pv : 0.f;
        if constexpr (DROP) {
          const float ks = drop_scale_of(pr, xb + (uint32_t)e * DROP_C_KEY);
          if constexpr (!TAN) dP[i] *= ks;
          if constexpr (DUAL || TAN) At[i] *= ks;
        }
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

    // ---- dQ^T += K^T dS^T (+ K'^T dS'^T): steps over (key chunk c, pair of d-blocks) -------------
    FragT tk[2][PW], tkt[2][PW];  // [ring slot][d-block of the group]
    auto issue_t = [&](auto ic) {
      constexpr int i = decltype(ic)::value, c = i / NDP, dp = i % NDP, sl = i % 2;
      constexpr int TO = (HB * 32 + c * 16) * ROWB;
#pragma unroll
      for (int u = 0; u < PW; ++u) {
        const uint32_t a0 = sbase + toff[PW * dp + u][0], a1 = sbase + toff[PW * dp + u][1];
        tk[sl][u].lo = lds_tr64<TO>(a0);
        tk[sl][u].hi = lds_tr64<TO>(a1);
        if constexpr (DUAL) {
          tkt[sl][u].lo = lds_tr64<TO + 2 * TILEB>(a0);
          tkt[sl][u].hi = lds_tr64<TO + 2 * TILEB>(a1);
        }
      }
    };
    constexpr int NRT = 2 * PW * NACC;
    issue_t(std::integral_constant<int, 0>{});
    static_for<NPV>([&](auto ic) {
      constexpr int i = decltype(ic)::value, c = i / NDP, dp = i % NDP, sl = i % 2;
      if constexpr (i + 1 < NPV) issue_t(std::integral_constant<int, i + 1>{});
      constexpr int younger = (i + 1 < NPV) ? NRT : 0;
      if constexpr (PW == 2) {
        if constexpr (DUAL) lds_wait<younger>(tk[sl][0], tk[sl][1], tkt[sl][0], tkt[sl][1]);
        else lds_wait<younger>(tk[sl][0], tk[sl][1]);
      } else {
        if constexpr (DUAL) lds_wait<younger>(tk[sl][0], tkt[sl][0]);
        else lds_wait<younger>(tk[sl][0].lo, tk[sl][0].hi);
      }
      load_step(std::integral_constant<int, 2 * KK + HB * NPV + i>{});
#pragma unroll
      for (int u = 0; u < PW; ++u) mma(acc[PW * dp + u], as_frag<T>(tk[sl][u]), dsf[c]);
      if constexpr (DUAL) {
#pragma unroll
        for (int u = 0; u < PW; ++u) mma(acc[PW * dp + u], as_frag<T>(tkt[sl][u]), dspf[c]);
      }
      if constexpr (SIX) {
#pragma unroll
        for (int u = 0; u < PW; ++u) mma(accT[PW * dp + u], as_frag<T>(tk[sl][u]), dspf[c]);
      }
    });
  };

  // Mask values travel from HBM or the far caches, further than one phase of matrix products hides:
  // those of tile t+1 are requested at the top of tile t.
  auto fetch_masks = [&](int tn) {
    if constexpr (MASK != MASK_NONE) {
      const int jn = tn * BT;
      if (mask_al && jn + BT <= Lk) {  // aligned rows, all 64 keys exist: one vector load per 8 keys
#pragma unroll
        for (int i = 0; i < 4; ++i) mnext[i / 2][i % 2] = mask_fetch8<T, MASK>(pr, mrow, jn + 16 * i + 8 * g);
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) mnext[i / 2][i % 2] = mask_fetch8_any<T, MASK>(pr, mrow, jn + 16 * i + 8 * g);
      }
    }
  };
  // the tile of this step and of the next
  int tcur = tlist ? min(max(tlist[1], 0), tmax) : 0;
  int tnext = tlist ? min(max(tlist[1 + min(1, ntiles - 1)], 0), tmax) : min(1, ntiles - 1);
  fetch_masks(tcur);
  prepare_loads(0, tcur * BT, true);
  static_for<NLOAD>([&](auto pc) { load_piece(pc); });
  auto tile = [&](int t, auto EDGEc) {
    const int j0 = tcur * BT;
    const int stage = t & 1;
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this wave's share of tile t has landed
    __syncthreads();                      // ... everyone's has, and stage^1 is no longer being read
    int tnext2 = min(t + 2, ntiles - 1), tahead = 0;
    if constexpr (MASK != MASK_NONE) {
      tahead = list_request(list_slot(tnext2));
#pragma unroll
      for (int i = 0; i < 4; ++i) mcur[i / 2][i % 2] = mnext[i / 2][i % 2];
      fetch_masks(tnext);
    }
    prepare_loads(stage ^ 1, tnext * BT, t + 1 < ntiles);
    const uint32_t sbase = lds0 + stage * Cfg::STAGEB;
    half_tile(std::integral_constant<int, 0>{}, EDGEc, sbase, j0);
    // always both halves: a half past the last key or past the diagonal contributes exact zeros, and a
    // branch here would make the accumulators change register file around it
    half_tile(std::integral_constant<int, 1>{}, EDGEc, sbase, j0 + 32);
    if constexpr (MASK != MASK_NONE) {
      const int listed = list_take(tahead);
      tnext2 = tlist ? min(max(listed, 0), tmax) : tnext2;
    }
    tcur = tnext;
    tnext = tnext2;
  };
  // Tiles that cross the diagonal or the end of the sequence are the last ones; they get a loop of their
  // own so that the common tile carries no limit tests.  (q0 is a multiple of the tile size.)
  int t_edge = Lk / BT;
  if (pr.causal) t_edge = min(t_edge, q0 / BT);
  if (MASK != MASK_NONE && !mask_al) t_edge = 0;  // interior tiles fetch mask rows with aligned vector loads
  int t = 0;
  if constexpr (!LEAN) {
    for (; t < ntiles && tcur < t_edge; ++t) tile(t, std::false_type{});
  }
  for (; t < ntiles; ++t) tile(t, std::true_type{});
  __builtin_amdgcn_s_waitcnt(0x0F70);  // the redirected loads of the last iteration must not outlive the kernel

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
        if constexpr (SIX) {
#pragma unroll
          for (int e = 0; e < 8; ++e) x[e] = accT[db][8 * hf + e] * pr.scale;
          store8<T>(reinterpret_cast<T *>(p.dqt) + head + (size_t)qrow * D + 32 * db + 16 * hf + 8 * g, x);
        }
      }
    }
  }
}
#endif
template <typename T, int D, int MODE, int MASK, bool GO, bool SIX = false, bool DROP = false>
__global__ __launch_bounds__(256, 1) void bwd2_dq_kernel(const BwdParams p) {
#if defined(__HIP_DEVICE_COMPILE__)
  bwd2_dq_body<T, D, MODE, MASK, GO, SIX, DROP>(p, blockIdx.x);
#endif
}
// The same code with the vector registers capped, for D = 64: together with the accumulation registers
// the kernel then needs at most 256 registers and two workgroups share a compute unit.
template <typename T, int D, int MODE, int MASK, bool GO, bool SIX = false>
__global__ __launch_bounds__(256, 1) __attribute__((amdgpu_num_vgpr(160))) void bwd2_dq_kernel_2wg(const BwdParams p) {
#if defined(__HIP_DEVICE_COMPILE__)
  bwd2_dq_body<T, D, MODE, MASK, GO, SIX>(p, blockIdx.x);
#endif
}

// D = 128 without tangents: Q, gO and the dq accumulator are 128 accumulation registers, so with the vector
// registers capped at 128 a wave stays within 256 and two workgroups (64 KB of LDS each) share a compute unit.
template <typename T, int D, int MODE, int MASK>
__global__ __launch_bounds__(256, 2) void bwd2_dq_kernel_2wg_plain(const BwdParams p) {
#if defined(__HIP_DEVICE_COMPILE__)
  static_assert(MODE == BWD_PLAIN && D == 128);
  bwd2_dq_body<T, D, MODE, MASK, true, false, false, MASK == MASK_NONE>(p, blockIdx.x);
#endif
}

// ------------------------------------------------------------------------------------------------
// dk, dv (PLAIN / DUAL) or dk', dv' (TANGENT): workgroup = 128 key rows, loop over 64-query tiles
// of Q, G (, Q', gT), G = gO (gT in TANGENT).  Scores are S = Q K^T (lane = key, registers =
// queries) so P, dS are the B operands of dV^T += G^T P and dK^T += Q^T dS.
#if defined(__HIP_DEVICE_COMPILE__)  // the host pass only needs the launch stubs (and has no buffer descriptor type)
// GROUPED: the key/value head serves several query heads (compiled apart, so that the common case of
// one keeps its pointers loop-invariant).
// SIX (dual mode only): dk' = scale dS'^T Q and dv' = P^T gT as well, from the fragments and tiles that dk, dv
// already have (two more accumulators: fits for D <= 64).
template <typename T, int D, int MODE, int MASK, bool GO, bool GROUPED, bool SIX, bool DROP = false>
__device__ __forceinline__ void bwd2_dkdv_body(const BwdParams &p, const int bid) {
  using Cfg = Bwd2Cfg<T, D, MODE>;
  constexpr bool DUAL = MODE == BWD_DUAL, TAN = MODE == BWD_TANGENT;
  static_assert(!SIX || (DUAL && D <= 64), "dk', dv' ride on the dual mode, where the accumulators fit");
  JVPFA_BWD2_COMMON(Cfg, pr.L, pr.Lk, pr.Hk)  // owns key rows (h: key/value head), streams query tiles
  const int kb = id % nblk;  // causal: the first key blocks have the longest query loops
  const int k0 = kb * Cfg::BLK;
  const int krow = k0 + wave * 32 + r;
  const int Lk = pr.Lk;  // keys; L counts queries
  const int kld = krow < Lk ? krow : Lk - 1;
  const uint32_t drop_lane = DROP ? (uint32_t)kld * DROP_C_KEY + (uint32_t)(8 * g) * DROP_C_ROW : 0u;
  if constexpr (MASK != MASK_NONE) {
    // a key block that the caller's hint declares fully masked has zero gradients
    if (pr.klimit && k0 >= pr.klimit[z]) {
      if (krow < Lk) {
        T *outk = reinterpret_cast<T *>(MODE == BWD_TANGENT ? p.dkt : p.dk) + head + (size_t)krow * D;
        T *outv = reinterpret_cast<T *>(MODE == BWD_TANGENT ? p.dvt : p.dv) + head + (size_t)krow * D;
        float zero8[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int d0 = 8 * g; d0 < D; d0 += 16) {
          store8<T>(outk + d0, zero8);
          store8<T>(outv + d0, zero8);
          if constexpr (SIX) {
            store8<T>(reinterpret_cast<T *>(p.dkt) + head + (size_t)krow * D + d0, zero8);
            store8<T>(reinterpret_cast<T *>(p.dvt) + head + (size_t)krow * D + d0, zero8);
          }
        }
      }
      return;
    }
  }
  constexpr bool has_go = GO;  // compile-time: a run-time test here would split every step into its own block
  const uint32_t stat0 = lds0 + 2 * Cfg::STAGEB;  // row statistics, two stages of NSTAT x 64 floats

  Frag<T> Kf[KK], Vf[KK], Ktf[DUAL ? KK : 1], Vtf[DUAL ? KK : 1];
  load_bfrags<KK>(Kf, reinterpret_cast<const T *>(p.k) + head + (size_t)kld * D, g);
  load_bfrags<KK>(Vf, reinterpret_cast<const T *>(p.v) + head + (size_t)kld * D, g);
  if constexpr (DUAL) {
    load_bfrags<KK>(Ktf, reinterpret_cast<const T *>(p.kt) + head + (size_t)kld * D, g);
    load_bfrags<KK>(Vtf, reinterpret_cast<const T *>(p.vt) + head + (size_t)kld * D, g);
  }
  // the resident operands live in the accumulation register file from here on
#pragma unroll
  for (int kk = 0; kk < KK; ++kk) {
    pin_acc(Kf[kk]);
    pin_acc(Vf[kk]);
    if constexpr (DUAL) {
      pin_acc(Ktf[kk]);  // V' stays in vector registers: the accumulation file also holds dK, dV
    }
  }

  f32x16 dK[DB], dV[DB], dKt[SIX ? DB : 1], dVt[SIX ? DB : 1];
#pragma unroll
  for (int db = 0; db < DB; ++db) {
    zero_acc(dK[db]);
    zero_acc(dV[db]);
    if constexpr (SIX) {
      zero_acc(dKt[db]);
      zero_acc(dVt[db]);
    }
  }

  const float sl2 = pr.scale * LOG2E;
  // mask element of (query 8g, this lane's key) relative to a row pointer, as a 32-bit offset
  bool mask_small = true;
  uint32_t mlane = 0;
  if constexpr (MASK != MASK_NONE) {
    const int64_t lim = (int64_t)1 << 31;
    mask_small = pr.ms[2] >= 0 && pr.ms[3] >= 0 && 8 * pr.ms[2] + (int64_t)Lk * pr.ms[3] < lim;
    mlane = (uint32_t)(8 * g * pr.ms[2] + (int64_t)kld * pr.ms[3]);
  }
  // MASK_TILE: the mask tile of (64 queries, this workgroup's 128 keys) is an operand tile of 256-byte rows in
  // all but name: direct loads with the chunks swizzled on the global side (wave w brings rows 16w .. 16w+15,
  // four instructions of four rows), and this lane's 16 values of a half tile (queries 16c + 8g + 0..7, its key)
  // come from the transposing fragment read of d-block `wave`.
  uint32_t mt_o[4] = {0u, 0u, 0u, 0u}, mt_f[2] = {0u, 0u};
  const uint32_t mt0 = lds0 + 2 * Cfg::STAGEB + 2 * Cfg::STATB;
  const char *mt_head = nullptr;       // first byte of (plane of the current query head, query 0, key k0)
  int64_t mt_row = 0;                  // bytes from a mask row to the next
  __amdgpu_buffer_rsrc_t mt_rs;
  uint32_t mt_dst = 0;
  if constexpr (MASK == MASK_TILE) {
    mt_row = pr.ms[2] * (int64_t)sizeof(T);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int row = 16 * wave + 4 * i + lane / 16;
      mt_o[i] = (uint32_t)(row * mt_row) + (uint32_t)(((lane % 16) ^ swz_u<16>(row)) * 16);
    }
    const int a_ = (lane >> 4) & 1, j_ = lane & 15;
#pragma unroll
    for (int hh = 0; hh < 2; ++hh) {
      const int row = 8 * g + 4 * hh + (j_ >> 2);
      // (the operand fragments take chunk j%2, half (j/2)%2, which hands lane r the column perm32(r); the mask
      // value must be that of the lane's own key, column r: chunk and half change places)
      mt_f[hh] = row * 256 + ((4 * wave + 2 * a_ + ((j_ >> 1) & 1)) ^ swz_u<16>(row)) * 16 + 8 * (j_ & 1);
    }
  }
  // The query heads that read this key/value head are visited one after another (one, h itself, for
  // the shapes the reference admits); hq is the current one, and what depends on it is set per head:
  // tile slots 0 Q, 1 G (gO; gT in TANGENT; gT again in DUAL without gO), 2 Q', 3 gT, and the
  // statistics slots PLAIN M, d1 | DUAL M, mu, a, d2 (= d1 + d2) | TANGENT M, a
  const int group = GROUPED ? pr.H / pr.Hk : 1;
  int hq = h * group;
  const char *Qb = nullptr, *gTb = nullptr, *Gb = nullptr, *Qtb = nullptr;
  const float *st_p[4] = {nullptr, nullptr, nullptr, nullptr};
  const uint32_t *bits_head = nullptr;  // MASK_BITS: the packed mask words of the current query head's plane
  auto set_query_head = [&](int hq_) {
    hq = hq_;
    const size_t qhead = ((size_t)z * pr.H + hq) * L * D * sizeof(T), qrow0 = ((size_t)z * pr.H + hq) * L;
    Qb = reinterpret_cast<const char *>(p.q) + qhead;
    gTb = (DUAL || TAN) ? reinterpret_cast<const char *>(p.gt) + qhead : nullptr;
    Gb = TAN ? gTb : (has_go ? reinterpret_cast<const char *>(p.go) + qhead : gTb);
    Qtb = DUAL ? reinterpret_cast<const char *>(p.qt) + qhead : nullptr;
    st_p[0] = p.M + qrow0;
    st_p[1] = MODE == BWD_PLAIN ? p.d1 + qrow0 : (DUAL ? p.mu + qrow0 : p.a + qrow0);
    st_p[2] = DUAL ? p.a + qrow0 : nullptr;
    st_p[3] = DUAL ? p.d2 + qrow0 : nullptr;
    if constexpr (MASK == MASK_BITS) bits_head = pr.bits_k + mask_bits_offset(pr, z, hq);
    if constexpr (MASK == MASK_TILE)
      mt_head = reinterpret_cast<const char *>(pr.mask) + (z * pr.ms[0] + hq * pr.ms[1] + (int64_t)k0) * (int64_t)sizeof(T);
  };
  set_query_head(h * group);

  const int istart = pr.causal ? (k0 / BT) * BT : 0;
  // Query tiles visited, counted from istart: 0 .. ntiles-1, or the caller's list of the tiles of this
  // key block that hold an attended entry (ascending; only with a mask, where istart is 0);
  // tile_at(i) is the i-th one.
  // The lists belong to the mask planes, one per query head: with grouped heads the list changes with
  // the head visited.
  const int *tlist = nullptr;
  const int tmax = (L + BT - 1) / BT - 1;  // index of the last tile of the sequence: bounds whatever a list holds
  int ntiles = (L - istart + BT - 1) / BT;
  auto set_list = [&](int hq_) {
    if constexpr (MASK != MASK_NONE) {
      if (pr.tiles_k) {
        tlist = pr.tiles_k + tile_list_offset_k(pr, z, hq_, kb);
        ntiles = min(max(tlist[0], 1), tmax + 1);
      }
    }
  };
  set_list(h * group);
  // List elements are requested a tile ahead, unconditionally (from a harmless address when there is
  // no list: a branch around the read would split the tile loop's straight-line body).
  auto list_slot = [&](int i) { return tlist ? tlist + 1 + i : reinterpret_cast<const int *>(p.q); };
  constexpr int NLOAD = IPW * Cfg::NTILE;
  constexpr int NPV = 2 * DB;  // accumulation steps of a half: (query chunk c, d-block db)
  constexpr int NSTEP = 2 * (KK + NPV);
  int st_row = 0;
  uint32_t st_dst = 0;
  auto prepare_loads = [&](int stage, int i0, bool on) {
    ld_dst = lds0 + stage * Cfg::STAGEB + (wave * IPW) * 1024;
    ld_rs[0] = tile_rsrc(Qb, i0, on);
    ld_rs[1] = tile_rsrc(Gb, i0, on);
    if constexpr (DUAL) {
      ld_rs[2] = tile_rsrc(Qtb, i0, on);
      ld_rs[3] = tile_rsrc(gTb, i0, on);
    }
    if constexpr (MASK == MASK_TILE) {
      // from (query i0, key k0) to the end of the last row's keys: rows past L and keys past Lk of the last
      // row read as zeros; keys past Lk of the other rows read the row that follows (lanes whose key does not
      // exist keep nothing)
      const int rows = on ? max(L - i0, 0) : 0;
      const int64_t bytes = rows > 0 ? (int64_t)(rows - 1) * mt_row + (int64_t)(Lk - k0) * (int64_t)sizeof(T) : 0;
      mt_rs = __builtin_amdgcn_make_buffer_rsrc((void *)(mt_head + (int64_t)i0 * mt_row), 0, (int)min(bytes, (int64_t)0x7fffffff), 0x00020000);
      mt_dst = mt0 + (Cfg::MTILE_SINGLE ? 0 : stage * Cfg::MTILEB) + (wave * 4) * 1024;
    }
    i0 = on ? i0 : istart;
    st_row = min(i0 + lane, L - 1);
    st_dst = stat0 + stage * Cfg::STATB;
  };
  // one 4-byte-per-lane direct load per statistic (64 rows); wave s loads statistic s
  auto load_stats = [&]() {
    if (wave < Cfg::NSTAT) {
      __builtin_amdgcn_global_load_lds((JVPFA_GLB(const void))(st_p[wave] + st_row),
                                       (JVPFA_LDS(void))(uintptr_t)(st_dst + wave * BT * 4), 4, 0, 0);
    }
  };
  // MASK_TILE: four more pieces per wave, rows 4i .. 4i+3 of the wave's 16
  constexpr int NLOAD_ALL = NLOAD + (MASK == MASK_TILE ? 4 : 0);
  auto load_any = [&](auto pc) {
    constexpr int pi = decltype(pc)::value;
    if constexpr (pi < NLOAD) {
      load_piece(pc);
    } else {
      constexpr int i = pi - NLOAD;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(mt_rs, (JVPFA_LDS(void))(uintptr_t)(mt_dst + i * 1024), 16, mt_o[i], 0, 0, 0);
    }
  };
  auto load_step = [&](auto gc) {
    constexpr int gi = decltype(gc)::value;
    // spread over the first NSPREAD steps only: the last load then has time to land before the barrier
    constexpr int NSPREAD = bwd_spread(NSTEP);
    if constexpr (gi < NSPREAD) {
      constexpr int lo = (gi * NLOAD_ALL + NSPREAD - 1) / NSPREAD, hi = ((gi + 1) * NLOAD_ALL + NSPREAD - 1) / NSPREAD;
      static_for<hi - lo>([&](auto dc) { load_any(std::integral_constant<int, lo + decltype(dc)::value>{}); });
    }
  };

  // EDGE: the half tile may cross the causal diagonal or the end of the sequence
  // Mask values of the half tile that starts at query ihn, for this lane's key.  They travel from HBM or
  // the far caches, so they are requested a whole half tile before their use.  (Where two workgroups
  // share a compute unit, D = 64 outside the dual mode, each value is instead fetched where it is used:
  // the other workgroup covers the wait and the registers stay within the cap.)
  constexpr bool MBYTES = MASK == MASK_BOOL || MASK == MASK_ADD;  // the mask itself, element by element
  constexpr bool MAHEAD = (D > 64 || MODE == BWD_DUAL) && MBYTES;
  T mnext_a[MASK == MASK_ADD ? 16 : 1];
  uint8_t mnext_b[MASK == MASK_BOOL ? 16 : 1];
  // MASK_BITS: this lane's key against the 64 queries of a tile is one pair of words (bit i of word hf = query
  // 32 hf + i of the tile).  The pair of the next tile is requested at the top of a tile, before any of the
  // tile's direct loads, and taken over behind the wait for everything at the top of the next one: the loop
  // body then holds no wait of its own for it (a wait in mid-tile would also wait for the direct loads issued
  // before it, which are meant to be in flight until the tile ends).
  u32x2 bits_next = {0u, 0u};
  auto fetch_bits = [&](int tile_index) {
    if constexpr (MASK == MASK_BITS)
      bits_next = *reinterpret_cast<const u32x2 *>(bits_head + ((size_t)tile_index * (size_t)Lk + (size_t)kld) * 2);
  };
  auto fetch_mask_half = [&](int ihn) {
    if constexpr (MBYTES) {
      if (mask_small && ihn + 32 <= L) {
        // uniform 64-bit row pointer + 32-bit lane offset: no per-lane address arithmetic per element
        const int64_t mrow0 = z * pr.ms[0] + hq * pr.ms[1];
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int64_t urow = mrow0 + (int64_t)(ihn + 16 * (e / 8) + (e % 8)) * pr.ms[2];
          if constexpr (MASK == MASK_ADD) mnext_a[e] = (reinterpret_cast<const T *>(pr.mask) + urow)[mlane];
          if constexpr (MASK == MASK_BOOL) mnext_b[e] = (reinterpret_cast<const uint8_t *>(pr.mask) + urow)[mlane];
        }
      } else {  // rows past the end are read from the last row (their scores are masked by index)
        const int64_t mcol = z * pr.ms[0] + hq * pr.ms[1] + (int64_t)kld * pr.ms[3];
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int qi = ihn + 16 * (e / 8) + 8 * g + (e % 8);
          const int64_t off = mcol + (int64_t)min(qi, L - 1) * pr.ms[2];
          if constexpr (MASK == MASK_ADD) mnext_a[e] = reinterpret_cast<const T *>(pr.mask)[off];
          if constexpr (MASK == MASK_BOOL) mnext_b[e] = reinterpret_cast<const uint8_t *>(pr.mask)[off];
        }
      }
    }
  };
  u32x2 mt_all[2][2][2];  // MASK_TILE with one stage: [half tile][chunk of 16 queries][4-row half]
  // ih: first query of this half tile; ihn: of the half tile that follows it
  auto half_tile = [&](auto HBc, auto EDGEc, uint32_t sbase, uint32_t sstat, int ih, int ihn, uint32_t bits_word, uint32_t mbase) {
    constexpr int HB = decltype(HBc)::value;
    // dropout: the 32 queries of a half tile are one block of the pattern (ih is a multiple of 32), so the block's
    // word is uniform and register e's query adds a constant to it; this lane's key and row group add drop_lane
    const uint32_t drop_half = DROP ? drop_row_word(pr, z * pr.H + hq, ih) + drop_lane : 0u;
    constexpr bool EDGE = decltype(EDGEc)::value;
    constexpr int RO = HB * 32 * ROWB;
    // ---- recompute ------------------------------------------------------------------------------
    // D = 64 reads fragments and statistics when it needs them instead of one step ahead: the
    // registers saved let two workgroups share a compute unit, and the second one covers the waits
    constexpr bool SAHEAD = D > 64;
    FragN fq[2], fg[2], fqt[2], fgt[2];
    auto issue_n = [&](auto kkc) {
      constexpr int kk = decltype(kkc)::value, sl = SAHEAD ? kk % 2 : 0;
      const uint32_t ad = sbase + noff[kk];
      fq[sl].v = lds_b128<RO>(ad);
      fg[sl].v = lds_b128<RO + TILEB>(ad);
      if constexpr (DUAL) {
        fqt[sl].v = lds_b128<RO + 2 * TILEB>(ad);
        fgt[sl].v = lds_b128<RO + 3 * TILEB>(ad);
      }
    };
    constexpr int NRN = DUAL ? 4 : 2;
    // mask values of this lane's key for the 32 queries of the half tile (register e <-> query
    // 16(e/8) + 8g + e%8): requested one half tile earlier (see fetch_mask_half), taken over here
    T mraw_a[MASK == MASK_ADD ? 16 : 1];
    uint8_t mraw_b[MASK == MASK_BOOL ? 16 : 1];
    const int64_t mcol_use = MASK != MASK_NONE ? z * pr.ms[0] + hq * pr.ms[1] + (int64_t)kld * pr.ms[3] : 0;
    // MASK_BITS: moved so that bit 16(e/8) + e%8 belongs to register e
    const uint32_t mraw_w = bits_word >> (8 * g);
    if constexpr (MASK != MASK_NONE && MAHEAD) {
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        if constexpr (MASK == MASK_ADD) mraw_a[e] = mnext_a[e];
        if constexpr (MASK == MASK_BOOL) mraw_b[e] = mnext_b[e];
      }
      fetch_mask_half(ihn);
    }
    // MASK_TILE: the 16 values of this half tile, four transposing reads issued ahead of every fragment read
    // of the half tile (LDS reads complete in order, so the first fragment wait covers them)
    u32x2 mtv[2][2];
    if constexpr (MASK == MASK_TILE && !Cfg::MTILE_SINGLE) {
      static_for<2>([&](auto cc) {
        constexpr int c = decltype(cc)::value, MO = (HB * 32 + c * 16) * 256;
        mtv[c][0] = lds_tr64<MO>(mbase + mt_f[0]);
        mtv[c][1] = lds_tr64<MO>(mbase + mt_f[1]);
      });
    }
    // tiles in ordinary vector registers; in DUAL, dP also collects gT V'^T (the B term)
    f32x16 S, dP, Sp, At;
    if constexpr (SAHEAD) issue_n(std::integral_constant<int, 0>{});
    static_for<KK>([&](auto kkc) {
      constexpr int kk = decltype(kkc)::value, sl = SAHEAD ? kk % 2 : 0;
      constexpr bool F = kk == 0;
      if constexpr (!SAHEAD) issue_n(std::integral_constant<int, kk>{});
      else if constexpr (kk + 1 < KK) issue_n(std::integral_constant<int, kk + 1>{});
      constexpr int younger_n = (SAHEAD && kk + 1 < KK) ? NRN : 0;
      if constexpr (DUAL) lds_wait<younger_n>(fq[sl], fg[sl], fqt[sl], fgt[sl]);
      else lds_wait<younger_n>(fq[sl], fg[sl]);
      load_step(std::integral_constant<int, HB * KK + kk>{});
      const Frag<T> q_ = as_frag<T>(fq[sl]), g_ = as_frag<T>(fg[sl]);
      mma_vra<F>(S, q_, Kf[kk]);
      if constexpr (MODE == BWD_PLAIN) mma_vra<F>(dP, g_, Vf[kk]);
      if constexpr (TAN) mma_vra<F>(At, g_, Vf[kk]);
      if constexpr (DUAL) {
        const Frag<T> gt_ = as_frag<T>(fgt[sl]);
        if constexpr (has_go) mma_vra<F>(dP, g_, Vf[kk]);
        mma_vra<F>(Sp, as_frag<T>(fqt[sl]), Kf[kk]);
        mma_vra<F>(At, gt_, Vf[kk]);
        mma_vra<false>(Sp, q_, Ktf[kk]);
        mma_vrv<F && !has_go>(dP, gt_, Vtf[kk]);
      }
    });
    if constexpr (DUAL) tiles_ready(S, dP, Sp, At);
    else if constexpr (TAN) tiles_ready(S, At);
    else tiles_ready(S, dP);

    // ---- row statistics of the 32 queries: register e belongs to query 16(e/8) + 8g + e%8 ------
    // read one quad of registers at a time (quad c4 = registers 4*c4 .. 4*c4+3), one quad ahead
    u32x4 stq[2][Cfg::NSTAT];
    const uint32_t sad = sstat + (HB * 32 + 8 * g) * 4;
    auto issue_s = [&](auto c4c) {
      constexpr int c4 = decltype(c4c)::value;
      static_for<Cfg::NSTAT>([&](auto sc) {
        constexpr int s_ = decltype(sc)::value;
        stq[c4 % 2][s_] = lds_b128<s_ * BT * 4 + (c4 / 2) * 64 + (c4 % 2) * 16>(sad);
      });
    };
    const int qmin = pr.causal ? krow : 0;  // queries below this index do not see this key
    // The 32 queries are handled as two chunks of 16 (registers 8c .. 8c+7): score gradients of a
    // chunk, then its share of dK^T += Q^T dS (+ Q'^T dS'), dV^T += G^T P (+ gT^T P'), one step per
    // d-block; the transposed fragments of a step are read one step ahead.
    FragT tq[2], tg[2], tqt[2], tgt[2];
    auto issue_t = [&](auto ic) {
      constexpr int i = decltype(ic)::value, c = i / DB, db = i % DB, sl = (D > 64) ? i % 2 : 0;
      constexpr int TO = (HB * 32 + c * 16) * ROWB;
      const uint32_t a0 = sbase + toff[db][0], a1 = sbase + toff[db][1];
      tq[sl].lo = lds_tr64<TO>(a0);
      tq[sl].hi = lds_tr64<TO>(a1);
      tg[sl].lo = lds_tr64<TO + TILEB>(a0);
      tg[sl].hi = lds_tr64<TO + TILEB>(a1);
      if constexpr (DUAL) {
        tqt[sl].lo = lds_tr64<TO + 2 * TILEB>(a0);
        tqt[sl].hi = lds_tr64<TO + 2 * TILEB>(a1);
        tgt[sl].lo = lds_tr64<TO + 3 * TILEB>(a0);
        tgt[sl].hi = lds_tr64<TO + 3 * TILEB>(a1);
      }
    };
    constexpr int NRT = DUAL ? 8 : 4;
    if constexpr (SAHEAD) issue_s(std::integral_constant<int, 0>{});
    Frag<T> mfr[2];
    if constexpr (MASK == MASK_TILE && Cfg::MTILE_SINGLE) {
      mfr[0] = as_frag<T>(FragT{mt_all[HB][0][0], mt_all[HB][0][1]});
      mfr[1] = as_frag<T>(FragT{mt_all[HB][1][0], mt_all[HB][1][1]});
    } else if constexpr (MASK == MASK_TILE) {
      lds_wait<SAHEAD ? Cfg::NSTAT : 0>(mtv[0][0], mtv[0][1], mtv[1][0], mtv[1][1]);  // long since there
      mfr[0] = as_frag<T>(FragT{mtv[0][0], mtv[0][1]});
      mfr[1] = as_frag<T>(FragT{mtv[1][0], mtv[1][1]});
    }
    static_for<2>([&](auto cc) {
      constexpr int c = decltype(cc)::value;
      f32x8 Pp;  // P * (S' - mu) of this chunk
      static_for<2>([&](auto hc) {
        constexpr int c4 = 2 * c + decltype(hc)::value, sl = c4 % 2;
        if constexpr (!SAHEAD) issue_s(std::integral_constant<int, c4>{});
        else if constexpr (c4 + 1 < 4) issue_s(std::integral_constant<int, c4 + 1>{});
        // waits also cover the transposed fragments issued before (LDS reads complete in order)
        constexpr int younger = (SAHEAD && c4 + 1 < 4) ? Cfg::NSTAT : 0;
        if constexpr (Cfg::NSTAT == 4) lds_wait4<younger>(stq[sl][0], stq[sl][1], stq[sl][2], stq[sl][3]);
        else lds_wait<younger>(stq[sl][0], stq[sl][1]);
        auto stat = [&](int s_, int e) { return __uint_as_float(stq[sl][s_][e % 4]); };
#pragma unroll
        for (int e = 4 * c4; e < 4 * c4 + 4; ++e) {
          const int qi = ih + 16 * (e / 8) + 8 * g + (e % 8);
          float s = S[e] * sl2;
          bool keep = true;
          if constexpr (MBYTES && !MAHEAD) {
            if constexpr (!EDGE) {  // uniform row pointer + 32-bit lane offset, as above
              const int64_t urow = z * pr.ms[0] + hq * pr.ms[1] + (int64_t)(ih + 16 * (e / 8) + (e % 8)) * pr.ms[2];
              if constexpr (MASK == MASK_ADD) mraw_a[0] = (reinterpret_cast<const T *>(pr.mask) + urow)[mlane];
              if constexpr (MASK == MASK_BOOL) mraw_b[0] = (reinterpret_cast<const uint8_t *>(pr.mask) + urow)[mlane];
            } else {
              const int64_t off = mcol_use + (int64_t)min(qi, L - 1) * pr.ms[2];
              if constexpr (MASK == MASK_ADD) mraw_a[0] = reinterpret_cast<const T *>(pr.mask)[off];
              if constexpr (MASK == MASK_BOOL) mraw_b[0] = reinterpret_cast<const uint8_t *>(pr.mask)[off];
            }
          }
          if constexpr (MASK == MASK_BOOL) keep = mraw_b[MAHEAD ? e : 0] != 0;
          // (additive: the mask value and the row's reference point in one term, the exponent one fused multiply-add)
          float pv;
          if constexpr (MASK == MASK_ADD) pv = fast_exp2(fmaf(S[e], sl2, fmaf((float)mraw_a[MAHEAD ? e : 0], LOG2E, -stat(0, e))));
          else if constexpr (MASK == MASK_TILE) pv = fast_exp2(fmaf(S[e], sl2, fmaf((float)mfr[e / 8][e % 8], LOG2E, -stat(0, e))));
          else pv = fast_exp2(s - stat(0, e));
          if constexpr (MASK == MASK_BOOL) pv = keep ? pv : 0.f;
          if constexpr (MASK == MASK_BITS) {
            // the entry's bit spread over a word (0 or all ones), and-ed onto P: two instructions (written as
            // asm: from the builtin the compiler makes a bit test, a compare and a select)
            uint32_t spread;
            asm("v_bfe_i32 %0, %1, %2, 1" : "=v"(spread) : "v"(mraw_w), "n"(16 * (e / 8) + (e % 8)));
            pv = __uint_as_float(__float_as_uint(pv) & spread);
          }
          if constexpr (EDGE) pv = (qi >= qmin && qi < L) ? pv : 0.f;
          float ks = 1.f;  // dropout: 1 / (1 - p) for a kept entry, 0 for a dropped one
          if constexpr (DROP) {
            ks = drop_scale_of(pr, drop_half + (uint32_t)(16 * (e / 8) + (e % 8)) * DROP_C_ROW);
            if constexpr (!TAN) dP[e] *= ks;
            if constexpr (DUAL || TAN) At[e] *= ks;
          }
          S[e] = pv * ks;
          if constexpr (MODE == BWD_PLAIN) {
            dP[e] = pv * (dP[e] - stat(1, e));
          } else if constexpr (DUAL) {
            const float sp = Sp[e] * pr.scale, m_ = stat(1, e), am = At[e] - stat(2, e);
            Pp[e - 8 * c] = pv * (sp - m_) * ks;
            Sp[e] = pv * am;
            dP[e] = pv * (dP[e] + am * sp - At[e] * m_ - stat(3, e));
          } else {
            Sp[e] = pv * (At[e] - stat(1, e));
          }
        }
      });
      const Frag<T> pf = to_frag<T>(S, c);
      Frag<T> dsf, dspf, ppf;
      if constexpr (!TAN) dsf = to_frag<T>(dP, c);
      if constexpr (DUAL || TAN) dspf = to_frag<T>(Sp, c);
      if constexpr (DUAL) {
#pragma unroll
        for (int e = 0; e < 8; ++e) ppf[e] = (T)Pp[e];
      }
      // the next quad of statistics (if any) was issued above, before these fragment reads
      if constexpr (SAHEAD) issue_t(std::integral_constant<int, c * DB>{});
      static_for<DB>([&](auto dbc) {
        constexpr int db = decltype(dbc)::value, i = c * DB + db, sl = SAHEAD ? i % 2 : 0;
        if constexpr (!SAHEAD) issue_t(std::integral_constant<int, i>{});
        else if constexpr (db + 1 < DB) issue_t(std::integral_constant<int, i + 1>{});
        constexpr int younger = (SAHEAD && db + 1 < DB) ? NRT : 0;
        if constexpr (DUAL) lds_wait<younger>(tq[sl], tg[sl], tqt[sl], tgt[sl]);
        else lds_wait<younger>(tq[sl], tg[sl]);
        load_step(std::integral_constant<int, 2 * KK + HB * NPV + i>{});
        if constexpr (MODE == BWD_PLAIN) {
          mma(dK[db], as_frag<T>(tq[sl]), dsf);
          mma(dV[db], as_frag<T>(tg[sl]), pf);
        } else if constexpr (DUAL) {
          mma(dK[db], as_frag<T>(tq[sl]), dsf);
          if constexpr (has_go) mma(dV[db], as_frag<T>(tg[sl]), pf);
          mma(dK[db], as_frag<T>(tqt[sl]), dspf);
          mma(dV[db], as_frag<T>(tgt[sl]), ppf);
          if constexpr (SIX) {
            mma(dKt[db], as_frag<T>(tq[sl]), dspf);
            mma(dVt[db], as_frag<T>(tgt[sl]), pf);
          }
        } else {
          mma(dK[db], as_frag<T>(tq[sl]), dspf);
          mma(dV[db], as_frag<T>(tg[sl]), pf);
        }
      });
    });
  };

  int tcur = 0, tnext = 0;  // the tile of this step and of the next
  auto tile = [&](int t, auto EDGEc) {
    const int stage = t & 1;
    __builtin_amdgcn_s_waitcnt(0x0F70);
    __syncthreads();
    if constexpr (MASK == MASK_TILE && Cfg::MTILE_SINGLE) {
      // the one stage of the mask tile: every wave takes its 32 values of this tile now; behind the second
      // barrier the stage belongs to the direct loads of the next tile
      static_for<4>([&](auto ic) {
        constexpr int hb = decltype(ic)::value / 2, c = decltype(ic)::value % 2, MO = (hb * 32 + c * 16) * 256;
        mt_all[hb][c][0] = lds_tr64<MO>(mt0 + mt_f[0]);
        mt_all[hb][c][1] = lds_tr64<MO>(mt0 + mt_f[1]);
      });
      asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier"
                   : "+v"(mt_all[0][0][0]), "+v"(mt_all[0][0][1]), "+v"(mt_all[0][1][0]), "+v"(mt_all[0][1][1]),
                     "+v"(mt_all[1][0][0]), "+v"(mt_all[1][0][1]), "+v"(mt_all[1][1][0]), "+v"(mt_all[1][1][1])
                   :
                   : "memory");
    }
    u32x2 bits_cur = bits_next;
    if constexpr (MASK == MASK_BITS) {
      asm volatile("" : "+v"(bits_cur));  // taken over here, behind the wait above
      fetch_bits(tnext);
    }
    int tnext2 = min(t + 2, ntiles - 1), tahead = 0;
    if constexpr (MASK != MASK_NONE) tahead = list_request(list_slot(tnext2));
    const int i0 = istart + tcur * BT, i0n = istart + tnext * BT;
    prepare_loads(stage ^ 1, i0n, t + 1 < ntiles);
    load_stats();
    const uint32_t sbase = lds0 + stage * Cfg::STAGEB, sstat = stat0 + stage * Cfg::STATB;
    const uint32_t mbase = mt0 + stage * Cfg::MTILEB;
    half_tile(std::integral_constant<int, 0>{}, EDGEc, sbase, sstat, i0, i0 + 32, bits_cur[0], mbase);
    // always both halves: a half past the last query contributes exact zeros, and a branch here would
    // make the accumulators change register file around it
    half_tile(std::integral_constant<int, 1>{}, EDGEc, sbase, sstat, i0 + 32, i0n, bits_cur[1], mbase);
    if constexpr (MASK != MASK_NONE) {
      const int listed = list_take(tahead);
      tnext2 = tlist ? min(max(listed, 0), tmax) : tnext2;
    }
    tcur = tnext;
    tnext = tnext2;
  };
  // Query tiles that cross the diagonal come first (causal), those that cross the end of the sequence
  // last; the tiles in between run without limit tests.
  const int t_diag = pr.causal ? min(ntiles, (k0 + Cfg::BLK - istart + BT - 1) / BT) : 0;
  const int t_end = mask_small ? max(t_diag, (L - istart) / BT) : t_diag;  // first tile that crosses the end
  for (int gi = 0; gi < group; ++gi) {
    if (gi > 0) {
      __syncthreads();  // every wave is done with the previous head's last tile: its stage may be refilled
      set_query_head(h * group + gi);
      if constexpr (GROUPED) set_list(h * group + gi);
    }
    tcur = tlist ? min(max(tlist[1], 0), tmax) : 0;
    tnext = tlist ? min(max(tlist[1 + min(1, ntiles - 1)], 0), tmax) : min(1, ntiles - 1);
    if constexpr (MASK != MASK_NONE && MAHEAD) fetch_mask_half(istart + tcur * BT);
    if constexpr (MASK == MASK_BITS) fetch_bits(tcur);
    prepare_loads(0, istart + tcur * BT, true);
    static_for<NLOAD_ALL>([&](auto pc) { load_any(pc); });
    load_stats();
    int t = 0;
    for (; t < t_diag; ++t) tile(t, std::true_type{});
    for (; t < ntiles && tcur < t_end; ++t) tile(t, std::false_type{});
    for (; t < ntiles; ++t) tile(t, std::true_type{});
    __builtin_amdgcn_s_waitcnt(0x0F70);
  }

  if (krow < Lk) {
    T *outk = reinterpret_cast<T *>(TAN ? p.dkt : p.dk) + head + (size_t)krow * D;
    T *outv = reinterpret_cast<T *>(TAN ? p.dvt : p.dv) + head + (size_t)krow * D;
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
        if constexpr (SIX) {
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            xk[e] = dKt[db][8 * hf + e] * pr.scale;
            xv[e] = dVt[db][8 * hf + e];
          }
          const size_t o = head + (size_t)krow * D + 32 * db + 16 * hf + 8 * g;
          store8<T>(reinterpret_cast<T *>(p.dkt) + o, xk);
          store8<T>(reinterpret_cast<T *>(p.dvt) + o, xv);
        }
      }
    }
  }
}
#endif
template <typename T, int D, int MODE, int MASK, bool GO, bool GROUPED = false, bool SIX = false, bool DROP = false>
__global__ __launch_bounds__(256, 1) void bwd2_dkdv_kernel(const BwdParams p) {
#if defined(__HIP_DEVICE_COMPILE__)
  bwd2_dkdv_body<T, D, MODE, MASK, GO, GROUPED, SIX, DROP>(p, blockIdx.x);
#endif
}
// The same code with the vector registers capped, for D = 64: together with the accumulation registers
// the kernel then needs at most 256 registers and two workgroups share a compute unit.
template <typename T, int D, int MODE, int MASK, bool GO, bool GROUPED = false>
__global__ __launch_bounds__(256, 1) __attribute__((amdgpu_num_vgpr(144))) void bwd2_dkdv_kernel_2wg(const BwdParams p) {
#if defined(__HIP_DEVICE_COMPILE__)
  bwd2_dkdv_body<T, D, MODE, MASK, GO, GROUPED, false>(p, blockIdx.x);
#endif
}

// Both roles in one launch, for grids smaller than the GPU: the first kv_blocks workgroups are dk/dv
// workgroups, the others dq workgroups.  The two kernels do not depend on each other, so launched apart on a
// stream each leaves the compute units it does not fill idle for its whole duration; together they run side
// by side.  (For grids that fill the GPU the single launch measured the same as the two.)
template <typename T, int D, int MODE, int MASK, bool GO>
__global__ __launch_bounds__(256, 1) void bwd2_both_kernel(const BwdParams p, const int kv_blocks) {
#if defined(__HIP_DEVICE_COMPILE__)
  const int b = __builtin_amdgcn_readfirstlane(blockIdx.x);
  if (b < kv_blocks) bwd2_dkdv_body<T, D, MODE, MASK, GO, false, false>(p, b);
  else bwd2_dq_body<T, D, MODE, MASK, GO, false>(p, b - kv_blocks);
#endif
}

}  // namespace jvpfa
