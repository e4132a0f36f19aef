// Backward kernels for 16-bit element types with D = 256 and no tangents in the launch (BWD_PLAIN: dq / dk, dv;
// BWD_TANGENT: dq' / dk', dv'), on the memory pipeline of bwd_kernel_v2.hpp.  (The dual mode has four resident
// operands instead of two and is built differently: bwd_kernel_pair.hpp.)
//
// The operands that stay in registers are 2 x 64 registers of the accumulation file (dq: Q and gO or gT; dk/dv:
// K and V); the accumulators cover all 256 columns (dq: 128 registers; dk and dv: 2 x 128).  Streamed tiles are
// 32 rows of 512 bytes: two stages of two 16 KB tiles; a tile is read both ways from its one row-major copy.
// The inline-asm matrix instructions are the guarded form (see mma_vra): with the accumulation file full the
// allocator moves resident operands through a spare register right before their use.
//
// First kernel: dq (PLAIN) or dq' (TANGENT).
#pragma once
#include "bwd_kernel_v2.hpp"

namespace jvpfa {

template <typename T, int D, int MODE> struct BwdWideCfg {
  static_assert(sizeof(T) == 2 && D == 256 && (MODE == BWD_PLAIN || MODE == BWD_TANGENT));
  static constexpr int NW = 4;
  static constexpr int NT = NW * WAVE;
  static constexpr int BLK = NW * 32;                 // rows owned by a workgroup
  static constexpr int BT = 32;                       // rows of a streamed tile
  static constexpr int CH = D * sizeof(T) / 16;       // 32 chunks of 16 bytes per row
  static constexpr int ROWB = D * sizeof(T);
  static constexpr int TILEB = BT * ROWB;
  static constexpr int NTILE = 2;
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
// DROP: dropout (see bwd_kernel.hpp): gO V^T (gT V^T) reaches the logits through the kept, rescaled entries only.
template <typename T, int D, int MODE, int MASK, bool DROP = false>
__global__ __launch_bounds__(256, 1) void bwdw_dq_kernel(const BwdParams p) {
  using Cfg = BwdWideCfg<T, D, MODE>;
  constexpr bool TAN = MODE == BWD_TANGENT;
  constexpr int CH = Cfg::CH, ROWB = Cfg::ROWB, TILEB = Cfg::TILEB, IPW = Cfg::IPW, BT = Cfg::BT;
  constexpr int KK = D / 16, DB = D / 32;
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
  const int r = lane % 32, g = lane / 32, pr32 = perm32(r);
  const size_t head = (size_t)zh * L * D;
  const size_t srow = (size_t)zh * L;
  const int q0 = qb * Cfg::BLK;
  const int qrow = q0 + wave * 32 + r;
  const int qld = qrow < L ? qrow : L - 1;

  // direct loads: instruction i of this wave fills LDS chunks 64*(wave*IPW+i) .. +63 of a tile
  uint32_t ld_o[IPW];
#pragma unroll
  for (int i = 0; i < IPW; ++i) {
    const int lc = 64 * (wave * IPW + i) + lane;
    const int row = lc / CH;
    ld_o[i] = row * ROWB + (((lc % CH) ^ swz_w(row)) * 16);
  }
  uint32_t ld_dst = 0;
  __amdgpu_buffer_rsrc_t ld_rs[2];
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
  // transposed fragment (see fwd_kernel_v2.hpp for the lane pattern): d-block db is at toff[db % 4] + 256 * (db / 4)
  uint32_t toff[4][2];
  {
    const int a_ = (lane >> 4) & 1, j_ = lane & 15;
#pragma unroll
    for (int db = 0; db < 4; ++db) {
#pragma unroll
      for (int hh = 0; hh < 2; ++hh) {
        const int row = 8 * g + 4 * hh + (j_ >> 2);
        const int ch = (4 * db + 2 * a_ + (j_ & 1)) ^ swz_w(row);
        toff[db][hh] = row * ROWB + ch * 16 + 8 * ((j_ >> 1) & 1);
      }
    }
  }

  // resident: Q and gO (PLAIN) or gT (TANGENT)
  Frag<T> Qf[KK], Gf[KK];
  load_bfrags<KK>(Qf, reinterpret_cast<const T *>(p.q) + head + (size_t)qld * D, g);
  load_bfrags<KK>(Gf, reinterpret_cast<const T *>(TAN ? p.gt : p.go) + head + (size_t)qld * D, g);
#pragma unroll
  for (int kk = 0; kk < KK; ++kk) {
    pin_acc(Qf[kk]);
    pin_acc(Gf[kk]);
  }

  const float Mq = qrow < L ? p.M[srow + qld] : __builtin_inff();
  const float sub = TAN ? p.a[srow + qld] : p.d1[srow + qld];  // what the row takes off dP (PLAIN) or A (TANGENT)
  const uint32_t drop_row = DROP ? drop_row_word(pr, zh, qld) : 0u;  // dropout: this lane's query row, see params.hpp

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

  int kend = pr.causal ? min(Lk, q0 + Cfg::BLK) : Lk;
  if constexpr (MASK != MASK_NONE) {
    if (pr.klimit) kend = min(kend, max(pr.klimit[z], 1));
  }
  // Key tiles visited: the 32-key tiles 0 .. ceil(kend/32)-1, or both halves of every 64-key tile of the
  // caller's list for this query block (the second half of the last one is dropped when it lies past
  // the last key).
  const int *tlist = nullptr;
  if constexpr (MASK != MASK_NONE) {
    if (pr.tiles_q) tlist = pr.tiles_q + tile_list_offset_q(pr, z, h, qb);
  }
  const int tmax = (Lk + TILE_W - 1) / TILE_W - 1;  // bounds whatever a list holds
  int ntiles = (kend + BT - 1) / BT;
  if (tlist) {
    const int cnt = min(max(tlist[0], 1), tmax + 1);
    const int last = min(max(tlist[cnt], 0), tmax);
    ntiles = 2 * cnt - (last * TILE_W + BT >= Lk ? 1 : 0);
  }
  auto list_slot = [&](int t) { return tlist ? tlist + 1 + (t >> 1) : reinterpret_cast<const int *>(p.q); };
  auto key_of = [&](int entry, int t) { return tlist ? min(max(entry, 0), tmax) * TILE_W + (t & 1) * BT : t * BT; };
  // tile slots in a stage: 0 K, 1 V
  constexpr int NLOAD = IPW * Cfg::NTILE;
  constexpr int NPV = 2 * (DB / 2);  // accumulation steps: (16-key chunk c, pair of d-blocks)
  constexpr int NSTEP = KK + NPV;
  auto prepare_loads = [&](int stage, int j0, bool on) {
    ld_dst = lds0 + stage * Cfg::STAGEB + (wave * IPW) * 1024;
    ld_rs[0] = tile_rsrc(Kb, j0, on);
    ld_rs[1] = tile_rsrc(Vb, j0, on);
  };
  auto load_step = [&](auto gc) {
    constexpr int gi = decltype(gc)::value;
    constexpr int NSPREAD = bwd_spread(NSTEP);
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
    // ---- recompute: S and dP = V gO^T (PLAIN) or A = V gT^T (TANGENT) ----------------------------
    FragN fk[2], fv[2];
    auto issue_n = [&](auto kkc) {
      constexpr int kk = decltype(kkc)::value, sl = kk % 2, HI = (kk / 8) * 256;
      const uint32_t ad = sbase + noff[kk % 8];
      fk[sl].v = lds_b128<HI>(ad);
      fv[sl].v = lds_b128<HI + TILEB>(ad);
    };
    f32x16 S, G;
    issue_n(std::integral_constant<int, 0>{});
    static_for<KK>([&](auto kkc) {
      constexpr int kk = decltype(kkc)::value, sl = kk % 2;
      constexpr bool F = kk == 0;
      if constexpr (kk + 1 < KK) issue_n(std::integral_constant<int, kk + 1>{});
      lds_wait<(kk + 1 < KK) ? 2 : 0>(fk[sl], fv[sl]);
      load_step(std::integral_constant<int, kk>{});
      mma_vra<F, true>(S, as_frag<T>(fk[sl]), Qf[kk]);
      mma_vra<F, true>(G, as_frag<T>(fv[sl]), Gf[kk]);
    });
    tiles_ready(S, G);

    // ---- P and the score gradient ---------------------------------------------------------------
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
        float gv = G[i];
        if constexpr (DROP) gv *= drop_scale_of(pr, drop_row + (uint32_t)(key0 + e) * DROP_C_KEY);
        S[i] = pv * (gv - sub);
      }
    }
    Frag<T> dsf[2];
#pragma unroll
    for (int c = 0; c < 2; ++c) dsf[c] = to_frag<T>(S, c);

    // ---- dQ^T += K^T dS^T -------------------------------------------------------------------------
    FragT tk[2][2];  // [ring slot][d-block of the pair]
    auto issue_t = [&](auto ic) {
      constexpr int i = decltype(ic)::value, c = i / (DB / 2), dp = i % (DB / 2), sl = i % 2;
      static_for<2>([&](auto uc) {
        constexpr int u = decltype(uc)::value, db = 2 * dp + u, TO = c * 16 * ROWB + (db / 4) * 256;
        const uint32_t a0 = sbase + toff[db % 4][0], a1 = sbase + toff[db % 4][1];
        tk[sl][u].lo = lds_tr64<TO>(a0);
        tk[sl][u].hi = lds_tr64<TO>(a1);
      });
    };
    issue_t(std::integral_constant<int, 0>{});
    static_for<NPV>([&](auto ic) {
      constexpr int i = decltype(ic)::value, c = i / (DB / 2), dp = i % (DB / 2), sl = i % 2;
      if constexpr (i + 1 < NPV) issue_t(std::integral_constant<int, i + 1>{});
      lds_wait<(i + 1 < NPV) ? 4 : 0>(tk[sl][0], tk[sl][1]);
      load_step(std::integral_constant<int, KK + i>{});
      mma(acc[2 * dp], as_frag<T>(tk[sl][0]), dsf[c]);
      mma(acc[2 * dp + 1], as_frag<T>(tk[sl][1]), dsf[c]);
    });
  };

  // mask values of tile t+1 are requested at the top of tile t
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
  // first keys of the tile of this step and of the next
  int jcur = key_of(tlist ? tlist[1] : 0, 0);
  int jnext = key_of(tlist ? tlist[1 + (min(1, ntiles - 1) >> 1)] : 0, min(1, ntiles - 1));
  fetch_masks(jcur);
  prepare_loads(0, jcur, true);
  static_for<NLOAD>([&](auto pc) { load_piece(pc); });
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
    int jnext2 = tnext2 * BT;
    if constexpr (MASK != MASK_NONE) jnext2 = key_of(list_take(tahead), tnext2);
    jcur = jnext;
    jnext = jnext2;
  };
  // tiles that cross the diagonal or the end of the sequence are the last ones
  int t_edge = Lk / BT;
  if (pr.causal) t_edge = min(t_edge, q0 / BT);
  if (MASK != MASK_NONE && !mask_al) t_edge = 0;
  int t = 0;
  for (; t < ntiles && jcur < t_edge * BT; ++t) tile(t, std::false_type{});
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
      }
    }
  }
}
#else
template <typename T, int D, int MODE, int MASK, bool DROP = false>
__global__ __launch_bounds__(256, 1) void bwdw_dq_kernel(const BwdParams p) {}
#endif

// ------------------------------------------------------------------------------------------------
// dk, dv (PLAIN) or dk', dv' (TANGENT) for D = 256: workgroup = 128 keys of a head, K and V resident,
// loop over 32-query tiles of Q and gO (PLAIN) or gT (TANGENT) with their row statistics.  With grouped
// heads the query heads that read this key/value head are visited one after another.
template <typename T, int D, int MODE> struct BwdWideKvCfg : BwdWideCfg<T, D, MODE> {
  static constexpr int NSTAT = 2;
  static constexpr int STATB = NSTAT * 64 * 4;  // 64 floats per statistic and stage (32 used)
  static constexpr size_t DKV_LDS = 2 * (size_t)BwdWideCfg<T, D, MODE>::STAGEB + 2 * (size_t)STATB;
};

#if defined(__HIP_DEVICE_COMPILE__)
template <typename T, int D, int MODE, int MASK, bool DROP = false>
__global__ __launch_bounds__(256, 1) void bwdw_dkdv_kernel(const BwdParams p) {
  using Cfg = BwdWideKvCfg<T, D, MODE>;
  constexpr bool TAN = MODE == BWD_TANGENT;
  constexpr int CH = Cfg::CH, ROWB = Cfg::ROWB, TILEB = Cfg::TILEB, IPW = Cfg::IPW, BT = Cfg::BT;
  constexpr int KK = D / 16, DB = D / 32;
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem_raw[];
  const uint32_t lds0 = (uint32_t)(uintptr_t)smem_raw;
  const Problem &pr = p.pr;
  const int L = pr.L, Lk = pr.Lk;  // queries, keys
  const int nblk = (Lk + Cfg::BLK - 1) / Cfg::BLK;
  const int id = xcd_remap(blockIdx.x, nblk, pr.Z * pr.Hk);
  const int zh = id / nblk;
  const int kb = id % nblk;  // causal: the first key blocks have the longest query loops
  const int z = zh / pr.Hk, hk = zh % pr.Hk, group = pr.H / pr.Hk;
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid / WAVE), lane = tid % WAVE;
  const int r = lane % 32, g = lane / 32, pr32 = perm32(r);
  const size_t head = (size_t)zh * Lk * D;   // of k, v and their gradients
  const int k0 = kb * Cfg::BLK;
  const int krow = k0 + wave * 32 + r;
  const int kld = krow < Lk ? krow : Lk - 1;
  const uint32_t drop_lane = DROP ? (uint32_t)kld * DROP_C_KEY + (uint32_t)(8 * g) * DROP_C_ROW : 0u;
  T *outk = reinterpret_cast<T *>(TAN ? p.dkt : p.dk) + head + (size_t)krow * D;
  T *outv = reinterpret_cast<T *>(TAN ? p.dvt : p.dv) + head + (size_t)krow * D;
  if constexpr (MASK != MASK_NONE) {
    // a key block that the caller's hint declares fully masked has zero gradients
    if (pr.klimit && k0 >= pr.klimit[z]) {
      if (krow < Lk) {
        float zero8[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int d0 = 8 * g; d0 < D; d0 += 16) {
          store8<T>(outk + d0, zero8);
          store8<T>(outv + d0, zero8);
        }
      }
      return;
    }
  }

  // direct loads of the streamed tiles, as in the dq kernel above
  uint32_t ld_o[IPW];
#pragma unroll
  for (int i = 0; i < IPW; ++i) {
    const int lc = 64 * (wave * IPW + i) + lane;
    const int row = lc / CH;
    ld_o[i] = row * ROWB + (((lc % CH) ^ swz_w(row)) * 16);
  }
  uint32_t ld_dst = 0;
  __amdgpu_buffer_rsrc_t ld_rs[2];
  auto tile_rsrc = [&](const char *base, int j, bool exists) {
    const int rows = exists ? max(L - j, 0) : 0;
    return __builtin_amdgcn_make_buffer_rsrc((void *)(base + (size_t)j * ROWB), 0, rows * ROWB, 0x00020000);
  };
  auto load_piece = [&](auto pc) {
    constexpr int pi = decltype(pc)::value, i = pi / Cfg::NTILE, ts = pi % Cfg::NTILE;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(ld_rs[ts], (JVPFA_LDS(void))(uintptr_t)(ld_dst + i * 1024 + ts * TILEB),
                                             16, ld_o[i], 0, 0, 0);
  };
  uint32_t noff[8];  // row-major fragment, steps kk and kk+8 differ by 256 bytes
  {
    const int x = swz_w(pr32);
#pragma unroll
    for (int kk = 0; kk < 8; ++kk) noff[kk] = pr32 * ROWB + (((2 * kk + g) ^ x) * 16);
  }
  // transposed fragment: d-block db is at toff[db % 4] + 256 * (db / 4)
  uint32_t toff[4][2];
  {
    const int a_ = (lane >> 4) & 1, j_ = lane & 15;
#pragma unroll
    for (int db = 0; db < 4; ++db) {
#pragma unroll
      for (int hh = 0; hh < 2; ++hh) {
        const int row = 8 * g + 4 * hh + (j_ >> 2);
        const int ch = (4 * db + 2 * a_ + (j_ & 1)) ^ swz_w(row);
        toff[db][hh] = row * ROWB + ch * 16 + 8 * ((j_ >> 1) & 1);
      }
    }
  }
  const uint32_t stat0 = lds0 + 2 * Cfg::STAGEB;  // row statistics, two stages of NSTAT x 64 floats

  Frag<T> Kf[KK], Vf[KK];
  load_bfrags<KK>(Kf, reinterpret_cast<const T *>(p.k) + head + (size_t)kld * D, g);
  load_bfrags<KK>(Vf, reinterpret_cast<const T *>(p.v) + head + (size_t)kld * D, g);
#pragma unroll
  for (int kk = 0; kk < KK; ++kk) {
    pin_acc(Kf[kk]);
    pin_acc(Vf[kk]);
  }

  f32x16 dK[DB], dV[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db) {
    zero_acc(dK[db]);
    zero_acc(dV[db]);
  }

  const float sl2 = pr.scale * LOG2E;
  bool mask_small = true;
  uint32_t mlane = 0;
  if constexpr (MASK != MASK_NONE) {
    const int64_t lim = (int64_t)1 << 31;
    mask_small = pr.ms[2] >= 0 && pr.ms[3] >= 0 && 8 * pr.ms[2] + (int64_t)Lk * pr.ms[3] < lim;
    mlane = (uint32_t)(8 * g * pr.ms[2] + (int64_t)kld * pr.ms[3]);
  }
  // tile slots 0 Q, 1 G (gO; gT in TANGENT), and the statistics slots PLAIN M, d1 | TANGENT M, a
  // h is the query head being visited; what depends on it is set per head
  int h = hk * group;
  const char *Qb = nullptr, *Gb = nullptr;
  const float *st_p[2] = {nullptr, nullptr};
  auto set_query_head = [&](int hq) {
    h = hq;
    const size_t qhead = ((size_t)z * pr.H + hq) * L * D * sizeof(T), srow = ((size_t)z * pr.H + hq) * L;
    Qb = reinterpret_cast<const char *>(p.q) + qhead;
    Gb = reinterpret_cast<const char *>(TAN ? p.gt : p.go) + qhead;
    st_p[0] = p.M + srow;
    st_p[1] = (TAN ? p.a : p.d1) + srow;
  };

  const int istart = pr.causal ? (k0 / BT) * BT : 0;
  // Query tiles visited, counted from istart: the 32-query tiles 0 .. ntiles-1, or both halves of every
  // 64-query tile of the caller's list for this key block and the query head visited (only with a
  // mask, where istart is 0); the second half of the last one is dropped when it lies past the end.
  const int *tlist = nullptr;
  const int tmax = (L + TILE_W - 1) / TILE_W - 1;  // bounds whatever a list holds
  int ntiles = (L - istart + BT - 1) / BT;
  auto set_list = [&](int hq) {
    if constexpr (MASK != MASK_NONE) {
      if (pr.tiles_k) {
        tlist = pr.tiles_k + tile_list_offset_k(pr, z, hq, kb);
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
  constexpr int NPV = 2 * DB;  // accumulation steps: (16-query chunk c, d-block db)
  constexpr int NSTEP = KK + NPV;
  int st_row = 0;
  uint32_t st_dst = 0;
  auto prepare_loads = [&](int stage, int i0, bool on) {
    ld_dst = lds0 + stage * Cfg::STAGEB + (wave * IPW) * 1024;
    ld_rs[0] = tile_rsrc(Qb, i0, on);
    ld_rs[1] = tile_rsrc(Gb, i0, on);
    i0 = on ? i0 : istart;
    st_row = min(i0 + lane, L - 1);
    st_dst = stat0 + stage * Cfg::STATB;
  };
  // one 4-byte-per-lane direct load per statistic (64 rows, the first 32 are the tile's); wave s loads statistic s
  auto load_stats = [&]() {
    if (wave < Cfg::NSTAT) {
      __builtin_amdgcn_global_load_lds((JVPFA_GLB(const void))(st_p[wave] + st_row),
                                       (JVPFA_LDS(void))(uintptr_t)(st_dst + wave * 64 * 4), 4, 0, 0);
    }
  };
  auto load_step = [&](auto gc) {
    constexpr int gi = decltype(gc)::value;
    constexpr int NSPREAD = bwd_spread(NSTEP);
    if constexpr (gi < NSPREAD) {
      constexpr int lo = (gi * NLOAD + NSPREAD - 1) / NSPREAD, hi = ((gi + 1) * NLOAD + NSPREAD - 1) / NSPREAD;
      static_for<hi - lo>([&](auto dc) { load_piece(std::integral_constant<int, lo + decltype(dc)::value>{}); });
    }
  };

  // mask values of the tile that starts at query ihn, for this lane's key, requested a tile ahead
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
      } else {  // rows past the end are read from the last row (their scores are masked by index)
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
  // ih: first query of this tile; ihn: of the tile that follows it
  auto tile_body = [&](auto EDGEc, uint32_t sbase, uint32_t sstat, int ih, int ihn) {
    constexpr bool EDGE = decltype(EDGEc)::value;
    // dropout: the 32 queries of a tile are one block of the pattern (ih is a multiple of 32), so the block's word
    // is uniform and register e's query adds a constant to it; this lane's key and row group add drop_lane
    const uint32_t drop_tile = DROP ? drop_row_word(pr, z * pr.H + h, ih) + drop_lane : 0u;
    // ---- recompute: S and dP = gO V^T (PLAIN) or A = gT V^T (TANGENT) -----------------------------
    FragN fq[2], fg[2];
    auto issue_n = [&](auto kkc) {
      constexpr int kk = decltype(kkc)::value, sl = kk % 2, HI = (kk / 8) * 256;
      const uint32_t ad = sbase + noff[kk % 8];
      fq[sl].v = lds_b128<HI>(ad);
      fg[sl].v = lds_b128<HI + TILEB>(ad);
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
    f32x16 S, G;
    issue_n(std::integral_constant<int, 0>{});
    static_for<KK>([&](auto kkc) {
      constexpr int kk = decltype(kkc)::value, sl = kk % 2;
      constexpr bool F = kk == 0;
      if constexpr (kk + 1 < KK) issue_n(std::integral_constant<int, kk + 1>{});
      lds_wait<(kk + 1 < KK) ? 2 : 0>(fq[sl], fg[sl]);
      load_step(std::integral_constant<int, kk>{});
      mma_vra<F, true>(S, as_frag<T>(fq[sl]), Kf[kk]);
      mma_vra<F, true>(G, as_frag<T>(fg[sl]), Vf[kk]);
    });
    tiles_ready(S, G);

    // ---- row statistics of the 32 queries: register e belongs to query 16(e/8) + 8g + e%8, read one
    // quad of registers at a time, one quad ahead
    u32x4 stq[2][Cfg::NSTAT];
    const uint32_t sad = sstat + 8 * g * 4;
    auto issue_s = [&](auto c4c) {
      constexpr int c4 = decltype(c4c)::value;
      static_for<Cfg::NSTAT>([&](auto sc) {
        constexpr int s_ = decltype(sc)::value;
        stq[c4 % 2][s_] = lds_b128<s_ * 64 * 4 + (c4 / 2) * 64 + (c4 % 2) * 16>(sad);
      });
    };
    const int qmin = pr.causal ? krow : 0;  // queries below this index do not see this key
    FragT tq[2], tg[2];
    // one step: transposed fragments of d-block db of chunk c; Q feeds dK, G feeds dV
    auto issue_t = [&](auto ic) {
      constexpr int i = decltype(ic)::value, c = i / DB, db = i % DB, sl = i % 2;
      constexpr int TO = c * 16 * ROWB + (db / 4) * 256;
      const uint32_t a0 = sbase + toff[db % 4][0], a1 = sbase + toff[db % 4][1];
      tq[sl].lo = lds_tr64<TO>(a0);
      tq[sl].hi = lds_tr64<TO>(a1);
      tg[sl].lo = lds_tr64<TO + TILEB>(a0);
      tg[sl].hi = lds_tr64<TO + TILEB>(a1);
    };
    issue_s(std::integral_constant<int, 0>{});
    static_for<2>([&](auto cc) {
      constexpr int c = decltype(cc)::value;
      static_for<2>([&](auto hc) {
        constexpr int c4 = 2 * c + decltype(hc)::value, sl = c4 % 2;
        if constexpr (c4 + 1 < 4) issue_s(std::integral_constant<int, c4 + 1>{});
        // waits also cover the transposed fragments issued before (LDS reads complete in order)
        lds_wait<(c4 + 1 < 4) ? Cfg::NSTAT : 0>(stq[sl][0], stq[sl][1]);
        auto stat = [&](int s_, int e) { return __uint_as_float(stq[sl][s_][e % 4]); };
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
          if constexpr (DROP) {
            const float ks = drop_scale_of(pr, drop_tile + (uint32_t)(16 * (e / 8) + (e % 8)) * DROP_C_ROW);
            S[e] = pv * ks;
            G[e] = pv * (G[e] * ks - stat(1, e));
          } else {
            S[e] = pv;
            G[e] = pv * (G[e] - stat(1, e));
          }
        }
      });
      const Frag<T> pf = to_frag<T>(S, c), dsf = to_frag<T>(G, c);
      issue_t(std::integral_constant<int, c * DB>{});
      static_for<DB>([&](auto dbc) {
        constexpr int db = decltype(dbc)::value, i = c * DB + db, sl = i % 2;
        if constexpr (db + 1 < DB) issue_t(std::integral_constant<int, i + 1>{});
        lds_wait<(db + 1 < DB) ? 4 : 0>(tq[sl], tg[sl]);
        load_step(std::integral_constant<int, KK + i>{});
        mma(dK[db], as_frag<T>(tq[sl]), dsf);
        mma(dV[db], as_frag<T>(tg[sl]), pf);
      });
    });
  };

  int icur = 0, inext = 0;  // first queries of the tile of this step and of the next
  auto tile = [&](int t, auto EDGEc) {
    const int stage = t & 1;
    __builtin_amdgcn_s_waitcnt(0x0F70);
    __syncthreads();
    const int tnext2 = min(t + 2, ntiles - 1);
    int tahead = 0;
    if constexpr (MASK != MASK_NONE) tahead = list_request(list_slot(tnext2));  // read a tile ahead
    prepare_loads(stage ^ 1, inext, t + 1 < ntiles);
    load_stats();
    tile_body(EDGEc, lds0 + stage * Cfg::STAGEB, stat0 + stage * Cfg::STATB, icur, inext);
    int inext2 = istart + tnext2 * BT;
    if constexpr (MASK != MASK_NONE) inext2 = query_of(list_take(tahead), tnext2);
    icur = inext;
    inext = inext2;
  };
  // Query tiles that cross the diagonal come first (causal), those that cross the end of the sequence
  // last; the tiles in between run without limit tests.
  const int t_diag = pr.causal ? min(ntiles, (k0 + Cfg::BLK - istart + BT - 1) / BT) : 0;
  const int t_end = mask_small ? max(t_diag, (L - istart) / BT) : t_diag;
  for (int gi = 0; gi < group; ++gi) {
    if (gi > 0) __syncthreads();  // every wave is done with the previous head's last tile: its stage may be refilled
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
#pragma unroll
    for (int db = 0; db < DB; ++db) {
#pragma unroll
      for (int hf = 0; hf < 2; ++hf) {
        float x[8], y[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          x[e] = dK[db][8 * hf + e] * pr.scale;
          y[e] = dV[db][8 * hf + e];
        }
        store8<T>(outk + 32 * db + 16 * hf + 8 * g, x);
        store8<T>(outv + 32 * db + 16 * hf + 8 * g, y);
      }
    }
  }
}
#else
template <typename T, int D, int MODE, int MASK, bool DROP = false>
__global__ __launch_bounds__(256, 1) void bwdw_dkdv_kernel(const BwdParams p) {}
#endif

}  // namespace jvpfa
