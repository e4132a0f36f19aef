// Dual-mode backward kernels for 16-bit element types with D = 256 in which two waves share 32 rows.
//
// bwd_kernel_wide.hpp keeps all four resident operands of a wave's 32 rows in its registers (4 x 64),
// which leaves room for the accumulators of half the output columns only, so two workgroups form every
// score tile.  Here the resident operands are split instead: the two waves of a pair own the same 32
// rows, each holds two of the four operands (2 x 64 registers), forms the score-sized tiles those two
// give, hands them to its partner through LDS and accumulates its share of the outputs.  Every product
// is then formed once (dq: 8 per tile instead of 14; dk, dv: 10 instead of 19).
//
//   dq     role 0 holds Q, Q'  and forms S = K Q^T,  S' = K Q'^T + K' Q^T
//          role 1 holds gT, gO and forms A = V gT^T, dP = V gO^T + V' gT^T
//          both take all four tiles from LDS, form dS, dS' (the same vector work twice) and accumulate
//          128 of dq's 256 columns each.
//   dk/dv  role 0 holds K, K'  and forms S, S';  P, P' follow and dV (all 256 columns) is its output
//          role 1 holds V, V'  and forms A, dP;  it takes S, S' from LDS, forms dS, dS' and accumulates dK.
//
// A workgroup is two pairs = 64 rows.  Streamed tiles, their swizzle, the direct loads and the fragment
// reads are those of bwd_kernel_wide.hpp; the tile slots are ordered so that the tiles of role 1 sit one
// slot behind those of role 0 and the two roles run the same instructions on different addresses.
// Mathematics and the reference lines replaced: see bwd_kernel.hpp.
#pragma once
#include "bwd_kernel_wide.hpp"

namespace jvpfa {

template <typename T, int D> struct BwdPairCfg {
  static_assert(sizeof(T) == 2 && D == 256);
  static constexpr int NW = 4;
  static constexpr int NT = NW * WAVE;
  static constexpr int BLK = 64;                      // rows owned by a workgroup: two pairs of waves
  static constexpr int BT = 32;                       // rows of a streamed tile
  static constexpr int DV = 128;                      // dq columns accumulated by one wave
  static constexpr int CH = D * sizeof(T) / 16;
  static constexpr int ROWB = D * sizeof(T);
  static constexpr int TILEB = BT * ROWB;
  static constexpr int NTILE = 4;
  static constexpr int STAGEB = NTILE * TILEB;
  static constexpr int IPW = TILEB / 1024 / NW;
  static constexpr int XTILE = WAVE * 16 * 4;         // one 32x32 fp32 tile as its owner's lanes hold it
  static constexpr int NSTAT = 4;
  static constexpr int STATB = NSTAT * 64 * 4;
  static constexpr size_t DQ_LDS = 2 * (size_t)STAGEB + 2 * 4 * (size_t)XTILE;                        // 160 KB
  static constexpr size_t DKV_LDS = 2 * (size_t)STAGEB + 2 * (size_t)STATB + 2 * 2 * (size_t)XTILE;   // 146 KB
};

// LDS traffic of the exchange, fixed in the program text like the fragment reads of pipeline.hpp.
template <int OFF> __device__ __forceinline__ void lds_put128(uint32_t addr, const f32x16 &x, int piece) {
  const f32x4 v = {x[4 * piece], x[4 * piece + 1], x[4 * piece + 2], x[4 * piece + 3]};
  asm volatile("ds_write_b128 %0, %1 offset:%2" : : "v"(addr), "v"(v), "n"(OFF) : "memory");
}
// this wave's LDS writes are done; then every wave of the workgroup has got here
__device__ __forceinline__ void exchange_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }
__device__ __forceinline__ void lds_wait_all(u32x4 (&a)[8]) {
  asm volatile("s_waitcnt lgkmcnt(0)"
               : "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3]), "+v"(a[4]), "+v"(a[5]), "+v"(a[6]), "+v"(a[7]));
}
__device__ __forceinline__ void lds_wait_all(u32x4 (&a)[16]) {
  asm volatile("s_waitcnt lgkmcnt(0)"
               : "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3]), "+v"(a[4]), "+v"(a[5]), "+v"(a[6]), "+v"(a[7]),
                 "+v"(a[8]), "+v"(a[9]), "+v"(a[10]), "+v"(a[11]), "+v"(a[12]), "+v"(a[13]), "+v"(a[14]), "+v"(a[15]));
}
// tile `slot` of an exchange area as the 16 accumulator registers of this lane
template <int SLOT, int N> __device__ __forceinline__ void xch_issue(u32x4 (&a)[N], uint32_t addr) {
  static_for<4>([&](auto jc) {
    constexpr int j = decltype(jc)::value;
    a[4 * SLOT + j] = lds_b128<j * 1024>(addr);
  });
}
template <int SLOT, int N> __device__ __forceinline__ f32x16 xch_tile(const u32x4 (&a)[N]) {
  f32x16 x;
#pragma unroll
  for (int e = 0; e < 16; ++e) x[e] = __uint_as_float(a[4 * SLOT + e / 4][e % 4]);
  return x;
}

#if defined(__HIP_DEVICE_COMPILE__)
// dq of the dual mode.  Tile slots of a stage: 0 K, 1 V, 2 K', 3 V'.
// SIX: dq' = scale dS' K as well, from the K fragments and the dS' tiles that dq already has (a call for all six
// gradients then needs no second launch that forms S and A again).
// DROP: dropout (see bwd_kernel.hpp): gO V^T, gT V^T and gT V'^T reach the logits through the kept, rescaled entries.
template <typename T, int D, int MASK, bool GO, bool SIX = false, bool DROP = false>
__global__ __launch_bounds__(256, 1) void bwdp_dq_kernel(const BwdParams p) {
  using Cfg = BwdPairCfg<T, D>;
  constexpr int CH = Cfg::CH, ROWB = Cfg::ROWB, TILEB = Cfg::TILEB, IPW = Cfg::IPW, BT = Cfg::BT, DV = Cfg::DV;
  constexpr int KK = D / 16, DB = DV / 32, XT = Cfg::XTILE;
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem_raw[];
  const uint32_t lds0 = (uint32_t)(uintptr_t)smem_raw;
  const Problem &pr = p.pr;
  const int L = pr.L;
  const int nblk = (L + Cfg::BLK - 1) / Cfg::BLK;
  const int id = xcd_remap(blockIdx.x, nblk, pr.Z * pr.H);
  const int zh = id / nblk;
  const int rem = id % nblk;
  const int qb = pr.causal ? nblk - 1 - rem : rem;
  const int z = zh / pr.H, h = zh % pr.H;
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid / WAVE), lane = tid % WAVE;
  const int pairi = wave >> 1, role = wave & 1;
  const int r = lane % 32, g = lane / 32, pr32 = perm32(r);
  const size_t head = (size_t)zh * L * D;
  const size_t srow = (size_t)zh * L;
  const int q0 = qb * Cfg::BLK;
  const int qrow = q0 + pairi * 32 + r;
  const int qld = qrow < L ? qrow : L - 1;

  uint32_t ld_o[IPW];
#pragma unroll
  for (int i = 0; i < IPW; ++i) {
    const int lc = 64 * (wave * IPW + i) + lane;
    const int row = lc / CH;
    ld_o[i] = row * ROWB + (((lc % CH) ^ swz_w(row)) * 16);
  }
  uint32_t ld_dst = 0;
  __amdgpu_buffer_rsrc_t ld_rs[4];
  auto tile_rsrc = [&](const char *base, int j, bool exists) {
    const int rows = exists ? max(pr.Lk - j, 0) : 0;
    return __builtin_amdgcn_make_buffer_rsrc((void *)(base + (size_t)j * ROWB), 0, rows * ROWB, 0x00020000);
  };
  auto load_piece = [&](auto pc) {
    constexpr int pi = decltype(pc)::value, i = pi / Cfg::NTILE, ts = pi % Cfg::NTILE;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(ld_rs[ts], (JVPFA_LDS(void))(uintptr_t)(ld_dst + i * 1024 + ts * TILEB),
                                             16, ld_o[i], 0, 0, 0);
  };
  // row-major fragments of this role's two tiles (slot role and slot role + 2)
  uint32_t noff[8];
  {
    const int x = swz_w(pr32);
#pragma unroll
    for (int kk = 0; kk < 8; ++kk) noff[kk] = role * TILEB + pr32 * ROWB + (((2 * kk + g) ^ x) * 16);
  }
  // transposed fragments of K, K' on this role's 128 columns
  uint32_t toff[DB][2];
  {
    const int a_ = (lane >> 4) & 1, j_ = lane & 15;
#pragma unroll
    for (int db = 0; db < DB; ++db) {
#pragma unroll
      for (int hh = 0; hh < 2; ++hh) {
        const int row = 8 * g + 4 * hh + (j_ >> 2);
        const int ch = (4 * db + 2 * a_ + (j_ & 1)) ^ swz_w(row);
        toff[db][hh] = row * ROWB + (16 * role + ch) * 16 + 8 * ((j_ >> 1) & 1);
      }
    }
  }
  // exchange area of this pair: tiles S, S', dP, A; role 0 writes the first two, role 1 the others
  const uint32_t xch = lds0 + 2 * Cfg::STAGEB + pairi * 4 * XT + lane * 16;
  const uint32_t xput_x = xch + (role ? 3 : 0) * XT, xput_y = xch + (role ? 2 : 1) * XT;

  // resident: role 0 A = Q, B = Q'; role 1 A = gT, B = gO (zeros when there is no gO)
  const T *arow = reinterpret_cast<const T *>(role ? p.gt : p.q) + head + (size_t)qld * D;
  const bool b_on = GO || role == 0;
  const T *brow = b_on ? reinterpret_cast<const T *>(role ? p.go : p.qt) + head + (size_t)qld * D : arow;
  Frag<T> Af[KK], Bf[KK];
  load_bfrags<KK>(Af, arow, g);
  load_bfrags<KK>(Bf, brow, g);
  if constexpr (!GO) {
    if (!b_on) {
#pragma unroll
      for (int kk = 0; kk < KK; ++kk) {
#pragma unroll
        for (int e = 0; e < 8; ++e) Bf[kk][e] = (T)0.f;
      }
    }
  }
#pragma unroll
  for (int kk = 0; kk < KK; ++kk) {
    pin_acc(Af[kk]);
    pin_acc(Bf[kk]);
  }

  const float Mq = qrow < L ? p.M[srow + qld] : __builtin_inff();
  const float mu = p.mu[srow + qld];
  const float av = p.a[srow + qld];
  const float dsum = p.d2[srow + qld];
  const uint32_t drop_row = DROP ? drop_row_word(pr, zh, qld) : 0u;  // dropout: this lane's query row, see params.hpp

  f32x16 acc[DB], accT[SIX ? DB : 1];
#pragma unroll
  for (int db = 0; db < DB; ++db) {
    zero_acc(acc[db]);
    if constexpr (SIX) zero_acc(accT[db]);
  }

  const float sl2 = pr.scale * LOG2E;
  const int64_t mrow = MASK != MASK_NONE ? z * pr.ms[0] + h * pr.ms[1] + (int64_t)qld * pr.ms[2] : 0;
  bool mask_al = false;
  if constexpr (MASK != MASK_NONE) mask_al = mask_rows_aligned<T, MASK>(pr);
  const int Lk = pr.Lk;
  const size_t kvhead = ((size_t)z * pr.Hk + h / (pr.H / pr.Hk)) * Lk * D;
  const char *Kb = reinterpret_cast<const char *>(p.k) + kvhead * sizeof(T);
  const char *Vb = reinterpret_cast<const char *>(p.v) + kvhead * sizeof(T);
  const char *Ktb = reinterpret_cast<const char *>(p.kt) + kvhead * sizeof(T);
  const char *Vtb = reinterpret_cast<const char *>(p.vt) + kvhead * sizeof(T);

  int kend = pr.causal ? min(Lk, q0 + Cfg::BLK) : Lk;
  if constexpr (MASK != MASK_NONE) {
    if (pr.klimit) kend = min(kend, max(pr.klimit[z], 1));
  }
  // Key tiles visited: the 32-key tiles 0 .. ceil(kend/32)-1, or both halves of every 64-key tile that the
  // caller's list names for the block of 128 query rows these 64 belong to.
  const int *tlist = nullptr;
  if constexpr (MASK != MASK_NONE) {
    if (pr.tiles_q) tlist = pr.tiles_q + tile_list_offset_q(pr, z, h, q0 / TILE_BLOCK);
  }
  const int tmax = (Lk + TILE_W - 1) / TILE_W - 1;
  int ntiles = (kend + BT - 1) / BT;
  if (tlist) {
    const int cnt = min(max(tlist[0], 1), tmax + 1);
    const int last = min(max(tlist[cnt], 0), tmax);
    ntiles = 2 * cnt - (last * TILE_W + BT >= Lk ? 1 : 0);
  }
  auto list_slot = [&](int t) { return tlist ? tlist + 1 + (t >> 1) : reinterpret_cast<const int *>(p.q); };
  auto key_of = [&](int entry, int t) { return tlist ? min(max(entry, 0), tmax) * TILE_W + (t & 1) * BT : t * BT; };
  constexpr int NLOAD = IPW * Cfg::NTILE;
  constexpr int NPV = 2 * (DB / 2);
  constexpr int NSTEP = KK + NPV;
  auto prepare_loads = [&](int stage, int j0, bool on) {
    ld_dst = lds0 + stage * Cfg::STAGEB + (wave * IPW) * 1024;
    ld_rs[0] = tile_rsrc(Kb, j0, on);
    ld_rs[1] = tile_rsrc(Vb, j0, on);
    ld_rs[2] = tile_rsrc(Ktb, j0, on);
    ld_rs[3] = tile_rsrc(Vtb, j0, on);
  };
  auto load_step = [&](auto gc) {
    constexpr int gi = decltype(gc)::value;
    constexpr int NSPREAD = bwd_spread(NSTEP);
    if constexpr (gi < NSPREAD) {
      constexpr int lo = (gi * NLOAD + NSPREAD - 1) / NSPREAD, hi = ((gi + 1) * NLOAD + NSPREAD - 1) / NSPREAD;
      static_for<hi - lo>([&](auto dc) { load_piece(std::integral_constant<int, lo + decltype(dc)::value>{}); });
    }
  };

  MaskAhead<T, MASK> mcur[2], mnext[2];
  const int klim = min(pr.causal ? qrow : 0x7fffffff, Lk - 1);
  auto tile_body = [&](auto EDGEc, uint32_t sbase, int j0) {
    constexpr bool EDGE = decltype(EDGEc)::value;
    // ---- this role's two tiles: X = f1 A, Y = f1 B + f2 A -----------------------------------------
    FragN f1[2], f2[2];
    auto issue_n = [&](auto kkc) {
      constexpr int kk = decltype(kkc)::value, sl = kk % 2, HI = (kk / 8) * 256;
      const uint32_t ad = sbase + noff[kk % 8];
      f1[sl].v = lds_b128<HI>(ad);
      f2[sl].v = lds_b128<HI + 2 * TILEB>(ad);
    };
    f32x16 X, Y;
    issue_n(std::integral_constant<int, 0>{});
    static_for<KK>([&](auto kkc) {
      constexpr int kk = decltype(kkc)::value, sl = kk % 2;
      constexpr bool F = kk == 0;
      if constexpr (kk + 1 < KK) issue_n(std::integral_constant<int, kk + 1>{});
      lds_wait<(kk + 1 < KK) ? 2 : 0>(f1[sl], f2[sl]);
      load_step(std::integral_constant<int, kk>{});
      const Frag<T> a_ = as_frag<T>(f1[sl]);
      mma_vra<F>(X, a_, Af[kk]);
      mma_vra<F>(Y, a_, Bf[kk]);
      mma_vra<false>(Y, as_frag<T>(f2[sl]), Af[kk]);
    });
    tiles_ready(X, Y);
    static_for<4>([&](auto jc) {
      constexpr int j = decltype(jc)::value;
      lds_put128<j * 1024>(xput_x, X, j);
      lds_put128<j * 1024>(xput_y, Y, j);
    });
    exchange_barrier();
    u32x4 xr[16];
    xch_issue<0>(xr, xch);
    xch_issue<1>(xr, xch + XT);
    xch_issue<2>(xr, xch + 2 * XT);
    xch_issue<3>(xr, xch + 3 * XT);
    lds_wait_all(xr);
    f32x16 S = xch_tile<0>(xr), Sp = xch_tile<1>(xr);
    const f32x16 dP = xch_tile<2>(xr), At = xch_tile<3>(xr);

    // ---- P and the score gradients (both waves of the pair) ---------------------------------------
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
        float dpv = dP[i], atv = At[i];
        if constexpr (DROP) {
          const float ks = drop_scale_of(pr, drop_row + (uint32_t)(key0 + e) * DROP_C_KEY);
          dpv *= ks;
          atv *= ks;
        }
        const float sp = Sp[i] * pr.scale, am = atv - av;
        Sp[i] = pv * am;
        S[i] = pv * (dpv + am * sp - atv * mu - dsum);
      }
    }
    Frag<T> dsf[2], dspf[2];
#pragma unroll
    for (int c = 0; c < 2; ++c) {
      dsf[c] = to_frag<T>(S, c);
      dspf[c] = to_frag<T>(Sp, c);
    }

    // ---- dQ^T += K^T dS^T + K'^T dS'^T on this role's columns -------------------------------------
    FragT tk[2][2], tkt[2][2];
    auto issue_t = [&](auto ic) {
      constexpr int i = decltype(ic)::value, c = i / (DB / 2), dp = i % (DB / 2), sl = i % 2;
      constexpr int TO = c * 16 * ROWB;
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const uint32_t a0 = sbase + toff[2 * dp + u][0], a1 = sbase + toff[2 * dp + u][1];
        tk[sl][u].lo = lds_tr64<TO>(a0);
        tk[sl][u].hi = lds_tr64<TO>(a1);
        tkt[sl][u].lo = lds_tr64<TO + 2 * TILEB>(a0);
        tkt[sl][u].hi = lds_tr64<TO + 2 * TILEB>(a1);
      }
    };
    issue_t(std::integral_constant<int, 0>{});
    static_for<NPV>([&](auto ic) {
      constexpr int i = decltype(ic)::value, c = i / (DB / 2), dp = i % (DB / 2), sl = i % 2;
      if constexpr (i + 1 < NPV) issue_t(std::integral_constant<int, i + 1>{});
      lds_wait<(i + 1 < NPV) ? 8 : 0>(tk[sl][0], tk[sl][1], tkt[sl][0], tkt[sl][1]);
      load_step(std::integral_constant<int, KK + i>{});
      mma(acc[2 * dp], as_frag<T>(tk[sl][0]), dsf[c]);
      mma(acc[2 * dp + 1], as_frag<T>(tk[sl][1]), dsf[c]);
      mma(acc[2 * dp], as_frag<T>(tkt[sl][0]), dspf[c]);
      mma(acc[2 * dp + 1], as_frag<T>(tkt[sl][1]), dspf[c]);
      if constexpr (SIX) {
        mma(accT[2 * dp], as_frag<T>(tk[sl][0]), dspf[c]);
        mma(accT[2 * dp + 1], as_frag<T>(tk[sl][1]), dspf[c]);
      }
    });
  };

  auto fetch_masks = [&](int jn) {
    if constexpr (MASK != MASK_NONE) {
      if (mask_al && jn + BT <= Lk) {
#pragma unroll
        for (int i = 0; i < 2; ++i) mnext[i] = mask_fetch8<T, MASK>(pr, mrow, jn + 16 * i + 8 * g);
      } else {
#pragma unroll
        for (int i = 0; i < 2; ++i) mnext[i] = mask_fetch8_any<T, MASK>(pr, mrow, jn + 16 * i + 8 * g);
      }
    }
  };
  int jcur = key_of(tlist ? tlist[1] : 0, 0);
  int jnext = key_of(tlist ? tlist[1 + (min(1, ntiles - 1) >> 1)] : 0, min(1, ntiles - 1));
  fetch_masks(jcur);
  prepare_loads(0, jcur, true);
  static_for<NLOAD>([&](auto pc) { load_piece(pc); });
  // Two barriers per tile.  The first: every wave's share of the tile has landed, nobody reads the other
  // stage any more, and the partner has taken the last tile's exchange (it reads it right behind the second
  // barrier, in front of its vector work).
  auto tile = [&](int t, auto EDGEc) {
    const int stage = t & 1;
    __builtin_amdgcn_s_waitcnt(0x0F70);
    __syncthreads();
    const int tnext2 = min(t + 2, ntiles - 1);
    int tahead = 0;
    if constexpr (MASK != MASK_NONE) {
      tahead = list_request(list_slot(tnext2));
      mcur[0] = mnext[0];
      mcur[1] = mnext[1];
      fetch_masks(jnext);
    }
    prepare_loads(stage ^ 1, jnext, t + 1 < ntiles);
    tile_body(EDGEc, lds0 + stage * Cfg::STAGEB, jcur);
    int jnext2 = tnext2 * BT;
    if constexpr (MASK != MASK_NONE) jnext2 = key_of(list_take(tahead), tnext2);
    jcur = jnext;
    jnext = jnext2;
  };
  int t_edge = Lk / BT;
  if (pr.causal) t_edge = min(t_edge, q0 / BT);
  if (MASK != MASK_NONE && !mask_al) t_edge = 0;
  int t = 0;
  for (; t < ntiles && jcur < t_edge * BT; ++t) tile(t, std::false_type{});
  for (; t < ntiles; ++t) tile(t, std::true_type{});
  __builtin_amdgcn_s_waitcnt(0x0F70);

  if (qrow < L) {
    T *out = reinterpret_cast<T *>(p.dq) + head + (size_t)qrow * D + role * DV;
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
          store8<T>(reinterpret_cast<T *>(p.dqt) + head + (size_t)qrow * D + role * DV + 32 * db + 16 * hf + 8 * g, x);
        }
      }
    }
  }
}

// dk, dv of the dual mode: workgroup = 64 keys of a key/value head (two pairs), loop over 32-query tiles.
// Tile slots of a stage: 0 Q, 1 gT, 2 Q', 3 gO; statistics slots M, mu, a, d2 (= d1 + d2).
template <typename T, int D, int MASK, bool GO, bool DROP = false>
__global__ __launch_bounds__(256, 1) void bwdp_dkdv_kernel(const BwdParams p) {
  using Cfg = BwdPairCfg<T, D>;
  constexpr int CH = Cfg::CH, ROWB = Cfg::ROWB, TILEB = Cfg::TILEB, IPW = Cfg::IPW, BT = Cfg::BT;
  constexpr int KK = D / 16, DB = D / 32, XT = Cfg::XTILE;
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem_raw[];
  const uint32_t lds0 = (uint32_t)(uintptr_t)smem_raw;
  const Problem &pr = p.pr;
  const int L = pr.L, Lk = pr.Lk;
  const int nblk = (Lk + Cfg::BLK - 1) / Cfg::BLK;
  const int id = xcd_remap(blockIdx.x, nblk, pr.Z * pr.Hk);
  const int zh = id / nblk;
  const int kb = id % nblk;
  const int z = zh / pr.Hk, hk = zh % pr.Hk, group = pr.H / pr.Hk;
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid / WAVE), lane = tid % WAVE;
  const int pairi = wave >> 1, role = wave & 1;
  const int r = lane % 32, g = lane / 32, pr32 = perm32(r);
  const size_t head = (size_t)zh * Lk * D;
  const int k0 = kb * Cfg::BLK;
  const int krow = k0 + pairi * 32 + r;
  const int kld = krow < Lk ? krow : Lk - 1;
  const uint32_t drop_lane = DROP ? (uint32_t)kld * DROP_C_KEY + (uint32_t)(8 * g) * DROP_C_ROW : 0u;
  // role 0 writes dV, role 1 dK
  T *out = reinterpret_cast<T *>(role ? p.dk : p.dv) + head + (size_t)krow * D;
  if constexpr (MASK != MASK_NONE) {
    if (pr.klimit && k0 >= pr.klimit[z]) {
      if (krow < Lk) {
        float zero8[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int d0 = 8 * g; d0 < D; d0 += 16) store8<T>(out + d0, zero8);
      }
      return;
    }
  }

  uint32_t ld_o[IPW];
#pragma unroll
  for (int i = 0; i < IPW; ++i) {
    const int lc = 64 * (wave * IPW + i) + lane;
    const int row = lc / CH;
    ld_o[i] = row * ROWB + (((lc % CH) ^ swz_w(row)) * 16);
  }
  uint32_t ld_dst = 0;
  __amdgpu_buffer_rsrc_t ld_rs[4];
  auto tile_rsrc = [&](const char *base, int j, bool exists) {
    const int rows = exists ? max(L - j, 0) : 0;
    return __builtin_amdgcn_make_buffer_rsrc((void *)(base + (size_t)j * ROWB), 0, rows * ROWB, 0x00020000);
  };
  auto load_piece = [&](auto pc) {
    constexpr int pi = decltype(pc)::value, i = pi / Cfg::NTILE, ts = pi % Cfg::NTILE;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(ld_rs[ts], (JVPFA_LDS(void))(uintptr_t)(ld_dst + i * 1024 + ts * TILEB),
                                             16, ld_o[i], 0, 0, 0);
  };
  // row-major fragments: role 0 reads Q (slot 0) and Q' (2), role 1 gT (1) and gO (3)
  uint32_t noff[8];
  {
    const int x = swz_w(pr32);
#pragma unroll
    for (int kk = 0; kk < 8; ++kk) noff[kk] = role * TILEB + pr32 * ROWB + (((2 * kk + g) ^ x) * 16);
  }
  // transposed fragments: role 0 (dV) reads gT (1) and gO (3), role 1 (dK) Q (0) and Q' (2); d-block db is at
  // toff[db % 4] + 256 * (db / 4)
  uint32_t toff[4][2];
  {
    const int a_ = (lane >> 4) & 1, j_ = lane & 15;
#pragma unroll
    for (int db = 0; db < 4; ++db) {
#pragma unroll
      for (int hh = 0; hh < 2; ++hh) {
        const int row = 8 * g + 4 * hh + (j_ >> 2);
        const int ch = (4 * db + 2 * a_ + (j_ & 1)) ^ swz_w(row);
        toff[db][hh] = (role ? 0 : TILEB) + row * ROWB + ch * 16 + 8 * ((j_ >> 1) & 1);
      }
    }
  }
  const uint32_t stat0 = lds0 + 2 * Cfg::STAGEB;
  // exchange area of this pair: S, S' as role 0's lanes hold them
  const uint32_t xch = stat0 + 2 * Cfg::STATB + pairi * 2 * XT + lane * 16;

  // resident: role 0 A = K, B = K'; role 1 A = V, B = V'
  Frag<T> Af[KK], Bf[KK];
  load_bfrags<KK>(Af, reinterpret_cast<const T *>(role ? p.v : p.k) + head + (size_t)kld * D, g);
  load_bfrags<KK>(Bf, reinterpret_cast<const T *>(role ? p.vt : p.kt) + head + (size_t)kld * D, g);
#pragma unroll
  for (int kk = 0; kk < KK; ++kk) {
    pin_acc(Af[kk]);
    pin_acc(Bf[kk]);
  }

  f32x16 acc[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db) zero_acc(acc[db]);

  const float sl2 = pr.scale * LOG2E;
  bool mask_small = true;
  uint32_t mlane = 0;
  if constexpr (MASK != MASK_NONE) {
    const int64_t lim = (int64_t)1 << 31;
    mask_small = pr.ms[2] >= 0 && pr.ms[3] >= 0 && 8 * pr.ms[2] + (int64_t)Lk * pr.ms[3] < lim;
    mlane = (uint32_t)(8 * g * pr.ms[2] + (int64_t)kld * pr.ms[3]);
  }
  int h = hk * group;
  const char *Qb = nullptr, *gTb = nullptr, *Gb = nullptr, *Qtb = nullptr;
  const float *st_p[4] = {nullptr, nullptr, nullptr, nullptr};
  auto set_query_head = [&](int hq) {
    h = hq;
    const size_t qhead = ((size_t)z * pr.H + hq) * L * D * sizeof(T), srow = ((size_t)z * pr.H + hq) * L;
    Qb = reinterpret_cast<const char *>(p.q) + qhead;
    gTb = reinterpret_cast<const char *>(p.gt) + qhead;
    Gb = GO ? reinterpret_cast<const char *>(p.go) + qhead : gTb;  // without gO the slot is loaded as zeros
    Qtb = reinterpret_cast<const char *>(p.qt) + qhead;
    st_p[0] = p.M + srow;
    st_p[1] = p.mu + srow;
    st_p[2] = p.a + srow;
    st_p[3] = p.d2 + srow;
  };

  const int istart = pr.causal ? (k0 / BT) * BT : 0;
  const int *tlist = nullptr;
  const int tmax = (L + TILE_W - 1) / TILE_W - 1;
  int ntiles = (L - istart + BT - 1) / BT;
  auto set_list = [&](int hq) {
    if constexpr (MASK != MASK_NONE) {
      if (pr.tiles_k) {  // the list of the block of 128 keys these 64 belong to
        tlist = pr.tiles_k + tile_list_offset_k(pr, z, hq, k0 / TILE_BLOCK);
        const int cnt = min(max(tlist[0], 1), tmax + 1);
        const int last = min(max(tlist[cnt], 0), tmax);
        ntiles = 2 * cnt - (last * TILE_W + BT >= L ? 1 : 0);
      }
    }
  };
  auto list_slot = [&](int t) { return tlist ? tlist + 1 + (t >> 1) : reinterpret_cast<const int *>(p.q); };
  auto query_of = [&](int entry, int t) {
    return tlist ? min(max(entry, 0), tmax) * TILE_W + (t & 1) * BT : istart + t * BT;
  };
  constexpr int NLOAD = IPW * Cfg::NTILE;
  constexpr int NPV = 2 * DB;
  constexpr int NSTEP = KK + NPV;
  int st_row = 0;
  uint32_t st_dst = 0;
  auto prepare_loads = [&](int stage, int i0, bool on) {
    ld_dst = lds0 + stage * Cfg::STAGEB + (wave * IPW) * 1024;
    ld_rs[0] = tile_rsrc(Qb, i0, on);
    ld_rs[1] = tile_rsrc(gTb, i0, on);
    ld_rs[2] = tile_rsrc(Qtb, i0, on);
    ld_rs[3] = tile_rsrc(Gb, i0, on && GO);
    i0 = on ? i0 : istart;
    st_row = min(i0 + lane, L - 1);
    st_dst = stat0 + stage * Cfg::STATB;
  };
  auto load_stats = [&]() {
    __builtin_amdgcn_global_load_lds((JVPFA_GLB(const void))(st_p[wave] + st_row),
                                     (JVPFA_LDS(void))(uintptr_t)(st_dst + wave * 64 * 4), 4, 0, 0);
  };
  auto load_step = [&](auto gc) {
    constexpr int gi = decltype(gc)::value;
    constexpr int NSPREAD = bwd_spread(NSTEP);
    if constexpr (gi < NSPREAD) {
      constexpr int lo = (gi * NLOAD + NSPREAD - 1) / NSPREAD, hi = ((gi + 1) * NLOAD + NSPREAD - 1) / NSPREAD;
      static_for<hi - lo>([&](auto dc) { load_piece(std::integral_constant<int, lo + decltype(dc)::value>{}); });
    }
  };

  T mnext_a[MASK == MASK_ADD ? 16 : 1];
  uint8_t mnext_b[MASK == MASK_BOOL ? 16 : 1];
  auto fetch_mask_tile = [&](int ihn) {
    if constexpr (MASK != MASK_NONE) {
      if (mask_small && ihn + 32 <= L) {
        const int64_t mrow0 = z * pr.ms[0] + h * pr.ms[1];
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int64_t urow = mrow0 + (int64_t)(ihn + 16 * (e / 8) + (e % 8)) * pr.ms[2];
          if constexpr (MASK == MASK_ADD) mnext_a[e] = (reinterpret_cast<const T *>(pr.mask) + urow)[mlane];
          if constexpr (MASK == MASK_BOOL) mnext_b[e] = (reinterpret_cast<const uint8_t *>(pr.mask) + urow)[mlane];
        }
      } else {
        const int64_t mcol = z * pr.ms[0] + h * pr.ms[1] + (int64_t)kld * pr.ms[3];
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
  auto tile_body = [&](auto EDGEc, uint32_t sbase, uint32_t sstat, int ih, int ihn) {
    constexpr bool EDGE = decltype(EDGEc)::value;
    // dropout: the 32 queries of a tile are one block of the pattern (ih is a multiple of 32), so the block's word
    // is uniform and register e's query adds a constant to it; this lane's key and row group add drop_lane
    const uint32_t drop_tile = DROP ? drop_row_word(pr, z * pr.H + h, ih) + drop_lane : 0u;
    // ---- this role's two tiles: X = f1 A, Y = f2 A + f1 B -----------------------------------------
    FragN f1[2], f2[2];
    auto issue_n = [&](auto kkc) {
      constexpr int kk = decltype(kkc)::value, sl = kk % 2, HI = (kk / 8) * 256;
      const uint32_t ad = sbase + noff[kk % 8];
      f1[sl].v = lds_b128<HI>(ad);
      f2[sl].v = lds_b128<HI + 2 * TILEB>(ad);
    };
    T mraw_a[MASK == MASK_ADD ? 16 : 1];
    uint8_t mraw_b[MASK == MASK_BOOL ? 16 : 1];
    if constexpr (MASK != MASK_NONE) {
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        if constexpr (MASK == MASK_ADD) mraw_a[e] = mnext_a[e];
        if constexpr (MASK == MASK_BOOL) mraw_b[e] = mnext_b[e];
      }
      fetch_mask_tile(ihn);
    }
    f32x16 X, Y;  // role 0: S, S'; role 1: A, dP (with the gT V'^T term)
    issue_n(std::integral_constant<int, 0>{});
    static_for<KK>([&](auto kkc) {
      constexpr int kk = decltype(kkc)::value, sl = kk % 2;
      constexpr bool F = kk == 0;
      if constexpr (kk + 1 < KK) issue_n(std::integral_constant<int, kk + 1>{});
      lds_wait<(kk + 1 < KK) ? 2 : 0>(f1[sl], f2[sl]);
      load_step(std::integral_constant<int, kk>{});
      const Frag<T> a_ = as_frag<T>(f1[sl]);
      mma_vra<F, true>(X, a_, Af[kk]);
      mma_vra<F, true>(Y, as_frag<T>(f2[sl]), Af[kk]);
      mma_vra<false, true>(Y, a_, Bf[kk]);
    });
    tiles_ready(X, Y);
    if (role == 0) {
      static_for<4>([&](auto jc) {
        constexpr int j = decltype(jc)::value;
        lds_put128<j * 1024>(xch, X, j);
        lds_put128<j * 1024>(xch + XT, Y, j);
      });
    }
    exchange_barrier();
    u32x4 xr[8];
    xch_issue<0>(xr, xch);
    xch_issue<1>(xr, xch + XT);
    lds_wait_all(xr);
    const f32x16 S = xch_tile<0>(xr), Sp = xch_tile<1>(xr);

    // ---- row statistics of the 32 queries, a quad of registers at a time, one quad ahead ----------
    u32x4 stq[2][4];
    const uint32_t sad = sstat + 8 * g * 4;
    auto issue_s = [&](auto c4c) {
      constexpr int c4 = decltype(c4c)::value;
      static_for<4>([&](auto sc) {
        constexpr int s_ = decltype(sc)::value;
        stq[c4 % 2][s_] = lds_b128<s_ * 64 * 4 + (c4 / 2) * 64 + (c4 % 2) * 16>(sad);
      });
    };
    const int qmin = pr.causal ? krow : 0;
    FragT ta[2], tb[2];
    const uint32_t tbase = sbase;
    auto issue_t = [&](auto ic) {
      constexpr int i = decltype(ic)::value, c = i / DB, db = i % DB, sl = i % 2;
      constexpr int TO = c * 16 * ROWB + (db / 4) * 256;
      const uint32_t a0 = tbase + toff[db % 4][0], a1 = tbase + toff[db % 4][1];
      ta[sl].lo = lds_tr64<TO>(a0);
      ta[sl].hi = lds_tr64<TO>(a1);
      tb[sl].lo = lds_tr64<TO + 2 * TILEB>(a0);
      tb[sl].hi = lds_tr64<TO + 2 * TILEB>(a1);
    };
    issue_s(std::integral_constant<int, 0>{});
    static_for<2>([&](auto cc) {
      constexpr int c = decltype(cc)::value;
      f32x8 Fa, Fb;  // role 0: P (S' - mu), P; role 1: dS, dS'
      static_for<2>([&](auto hc) {
        constexpr int c4 = 2 * c + decltype(hc)::value, sl = c4 % 2;
        if constexpr (c4 + 1 < 4) issue_s(std::integral_constant<int, c4 + 1>{});
        constexpr int younger = (c4 + 1 < 4) ? 4 : 0;
        lds_wait4<younger>(stq[sl][0], stq[sl][1], stq[sl][2], stq[sl][3]);
        auto stat = [&](int s_, int e) { return __uint_as_float(stq[sl][s_][e % 4]); };
        float pv4[4], sp4[4], ks4[4];
#pragma unroll
        for (int e = 4 * c4; e < 4 * c4 + 4; ++e) {
          const int qi = ih + 16 * (e / 8) + 8 * g + (e % 8);
          float s = S[e] * sl2;
          bool keep = true;
          if constexpr (MASK == MASK_ADD) s += (float)mraw_a[e] * LOG2E;
          if constexpr (MASK == MASK_BOOL) keep = mraw_b[e] != 0;
          float pv = fast_exp2(s - stat(0, e));
          if constexpr (MASK == MASK_BOOL) pv = keep ? pv : 0.f;
          if constexpr (EDGE) pv = (qi >= qmin && qi < L) ? pv : 0.f;
          pv4[e % 4] = pv;
          sp4[e % 4] = Sp[e] * pr.scale;
          ks4[e % 4] = DROP ? drop_scale_of(pr, drop_tile + (uint32_t)(16 * (e / 8) + (e % 8)) * DROP_C_ROW) : 1.f;
        }
        if (role) {  // X = A, Y = dP
#pragma unroll
          for (int e = 4 * c4; e < 4 * c4 + 4; ++e) {
            const float at = DROP ? X[e] * ks4[e % 4] : X[e], dp = DROP ? Y[e] * ks4[e % 4] : Y[e];
            const float pv = pv4[e % 4], m_ = stat(1, e), am = at - stat(2, e);
            Fa[e - 8 * c] = pv * (dp + am * sp4[e % 4] - at * m_ - stat(3, e));
            Fb[e - 8 * c] = pv * am;
          }
        } else {
#pragma unroll
          for (int e = 4 * c4; e < 4 * c4 + 4; ++e) {
            const float pw = DROP ? pv4[e % 4] * ks4[e % 4] : pv4[e % 4];
            Fa[e - 8 * c] = pw * (sp4[e % 4] - stat(1, e));
            Fb[e - 8 * c] = pw;
          }
        }
      });
      Frag<T> fa, fb;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        fa[e] = (T)Fa[e];
        fb[e] = (T)Fb[e];
      }
      issue_t(std::integral_constant<int, c * DB>{});
      static_for<DB>([&](auto dbc) {
        constexpr int db = decltype(dbc)::value, i = c * DB + db, sl = i % 2;
        if constexpr (db + 1 < DB) issue_t(std::integral_constant<int, i + 1>{});
        lds_wait<(db + 1 < DB) ? 4 : 0>(ta[sl], tb[sl]);
        load_step(std::integral_constant<int, KK + i>{});
        // role 0: dV += gT^T P (S' - mu) + gO^T P; role 1: dK += Q^T dS + Q'^T dS'
        mma(acc[db], as_frag<T>(ta[sl]), fa);
        mma(acc[db], as_frag<T>(tb[sl]), fb);
      });
    });
  };

  int icur = 0, inext = 0;
  auto tile = [&](int t, auto EDGEc) {
    const int stage = t & 1;
    __builtin_amdgcn_s_waitcnt(0x0F70);
    __syncthreads();
    const int tnext2 = min(t + 2, ntiles - 1);
    int tahead = 0;
    if constexpr (MASK != MASK_NONE) tahead = list_request(list_slot(tnext2));
    prepare_loads(stage ^ 1, inext, t + 1 < ntiles);
    load_stats();
    tile_body(EDGEc, lds0 + stage * Cfg::STAGEB, stat0 + stage * Cfg::STATB, icur, inext);
    int inext2 = istart + tnext2 * BT;
    if constexpr (MASK != MASK_NONE) inext2 = query_of(list_take(tahead), tnext2);
    icur = inext;
    inext = inext2;
  };
  const int t_diag = pr.causal ? min(ntiles, (k0 + Cfg::BLK - istart + BT - 1) / BT) : 0;
  const int t_end = mask_small ? max(t_diag, (L - istart) / BT) : t_diag;
  for (int gi = 0; gi < group; ++gi) {
    if (gi > 0) __syncthreads();
    set_query_head(hk * group + gi);
    set_list(hk * group + gi);
    icur = query_of(tlist ? tlist[1] : 0, 0);
    inext = query_of(tlist ? tlist[1 + (min(1, ntiles - 1) >> 1)] : 0, min(1, ntiles - 1));
    if constexpr (MASK != MASK_NONE) fetch_mask_tile(icur);
    prepare_loads(0, icur, true);
    static_for<NLOAD>([&](auto pc) { load_piece(pc); });
    load_stats();
    int t = 0;
    for (; t < t_diag; ++t) tile(t, std::true_type{});
    for (; t < ntiles && icur < istart + t_end * BT; ++t) tile(t, std::false_type{});
    for (; t < ntiles; ++t) tile(t, std::true_type{});
    __builtin_amdgcn_s_waitcnt(0x0F70);
  }

  if (krow < Lk) {
    const float os = role ? pr.scale : 1.f;
#pragma unroll
    for (int db = 0; db < DB; ++db) {
#pragma unroll
      for (int hf = 0; hf < 2; ++hf) {
        float x[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) x[e] = acc[db][8 * hf + e] * os;
        store8<T>(out + 32 * db + 16 * hf + 8 * g, x);
      }
    }
  }
}
#else
template <typename T, int D, int MASK, bool GO, bool SIX = false, bool DROP = false>
__global__ __launch_bounds__(256, 1) void bwdp_dq_kernel(const BwdParams p) {}
template <typename T, int D, int MASK, bool GO, bool DROP = false>
__global__ __launch_bounds__(256, 1) void bwdp_dkdv_kernel(const BwdParams p) {}
#endif

}  // namespace jvpfa
