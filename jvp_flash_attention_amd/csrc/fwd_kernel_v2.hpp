// Fused dual forward for 16-bit element types (bf16 / fp16), D in {64, 128}: the headline kernel.
//
// Same mathematics and register layout as fwd_kernel.hpp (one workgroup = 4 waves = 128 query
// rows, scores formed transposed so that a lane owns a query column), with the memory side
// rebuilt for gfx950:
//   * K, K', V, V' tiles (64 keys) go global -> LDS with direct-to-LDS loads (no registers, no
//     VALU), double buffered: the loads of tile j+1 are in flight while tile j is computed, and
//     there is one workgroup barrier per tile.
//   * every tile is stored row-major; 16-byte chunks are XOR-swizzled on the global-address side
//     so that both read patterns below are bank-conflict free without padding.
//   * K / K' fragments (contraction over d) are read with ds_read_b128; V / V' fragments
//     (contraction over keys) with the transposing ds_read_b64_tr_b16, so V is never transposed
//     in memory.
#pragma once
#include <utility>

#include "common.hpp"
#include "mask.hpp"
#include "params.hpp"
#include "pipeline.hpp"

namespace jvpfa {

template <typename T, int D, bool DUAL> struct Fwd2Cfg {
  static constexpr int NW = 4;
  static constexpr int NT = NW * WAVE;
  static constexpr int BM = NW * 32;
  static constexpr int BN = 64;
  static constexpr int CH = D * sizeof(T) / 16;       // 16-byte chunks per row
  static constexpr int ROWB = D * sizeof(T);          // bytes per row
  static constexpr int TILEB = BN * ROWB;             // bytes per tile
  static constexpr int NTILE = DUAL ? 4 : 2;          // K, V (, K', V')
  static constexpr int STAGEB = NTILE * TILEB;
  static constexpr size_t LDS_BYTES = 2 * (size_t)STAGEB;
  static constexpr int IPW = TILEB / 1024 / NW;       // direct-load instructions per wave per tile
};

// DROP: dropout on the probabilities (see fwd_kernel.hpp): what enters the products with V, V' is
// P * keep / (1 - p); the row sums l, mu stay those of the full softmax.
template <typename T, int D, bool DUAL, int MASK, bool DROP = false>
__global__ __launch_bounds__(256, 1) void fwd2_kernel(const FwdParams p) {
  using Cfg = Fwd2Cfg<T, D, DUAL>;
  constexpr int BN = Cfg::BN, CH = Cfg::CH, ROWB = Cfg::ROWB, TILEB = Cfg::TILEB, IPW = Cfg::IPW;
  constexpr int NB = BN / 32, KK = D / 16, DB = D / 32;
  constexpr float NEG_INF = -__builtin_inff();

  extern __shared__ __attribute__((aligned(1024))) unsigned char smem_raw[];
  // stage s: [K | V | K' | V'] each TILEB bytes
  const uint32_t lds0 = (uint32_t)(uintptr_t)smem_raw;

  const Problem &pr = p.pr;
  const int L = pr.L;
  const int nqb = (L + Cfg::BM - 1) / Cfg::BM;
  const int total = nqb * pr.Z * pr.H;
  const int id = xcd_remap(blockIdx.x, nqb, pr.Z * pr.H);
  const int zh = id / nqb;
  const int qb = pr.causal ? nqb - 1 - id % nqb : id % nqb;
  const int z = zh / pr.H, h = zh % pr.H;

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid / WAVE), lane = tid % WAVE;  // wave index is uniform
  const int r = lane % 32, g = lane / 32;
  const int pr32 = perm32(r);

  const size_t head = (size_t)zh * L * D;
  // keys: Lk of them, in head h / (H / Hk) of the key/value tensors (L and h themselves for the
  // shapes the reference admits)
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
  // 64*(wave*IPW+i) .. +63 of a tile; this lane's chunk holds (row, logical chunk c).
  // Byte offsets inside a full tile are per-lane constants, so a load is "uniform tile pointer +
  // 32-bit lane offset"; only a ragged last tile recomputes them with the row clamped to L-1.
  int ld_row[IPW];
  uint32_t ld_ck[IPW], ld_cv[IPW], ld_bk[IPW], ld_bv[IPW];
#pragma unroll
  for (int i = 0; i < IPW; ++i) {
    const int lc = 64 * (wave * IPW + i) + lane;
    const int row = lc / CH, cp = lc % CH;
    ld_row[i] = row;
    ld_ck[i] = (cp ^ swz_k<CH>(row)) * 16;  // byte offset within the row, K-type tiles
    ld_cv[i] = (cp ^ swz_v<CH>(row)) * 16;  // V-type tiles
    ld_bk[i] = row * ROWB + ld_ck[i];
    ld_bv[i] = row * ROWB + ld_cv[i];
  }
  auto issue_loads = [&](int stage, int j0) {
    const uint32_t sbase = lds0 + stage * Cfg::STAGEB + (wave * IPW) * 1024;
    const size_t tb = (size_t)j0 * ROWB;
    const char *kp = reinterpret_cast<const char *>(Kg) + tb, *vp = reinterpret_cast<const char *>(Vg) + tb;
    const char *ktp = DUAL ? reinterpret_cast<const char *>(Ktg) + tb : nullptr;
    const char *vtp = DUAL ? reinterpret_cast<const char *>(Vtg) + tb : nullptr;
    const bool ragged_tile = j0 + BN > Lk;
#pragma unroll
    for (int i = 0; i < IPW; ++i) {
      uint32_t ok = ld_bk[i], ov = ld_bv[i];
      if (ragged_tile) {  // rows past the end re-read the last row; their scores are masked
        const int row = min(ld_row[i], Lk - 1 - j0);
        ok = row * ROWB + ld_ck[i];
        ov = row * ROWB + ld_cv[i];
      }
      const uint32_t dst = sbase + i * 1024;
      __builtin_amdgcn_global_load_lds((JVPFA_GLB(const void))(kp + ok), (JVPFA_LDS(void))(uintptr_t)(dst), 16, 0, 0);
      __builtin_amdgcn_global_load_lds((JVPFA_GLB(const void))(vp + ov), (JVPFA_LDS(void))(uintptr_t)(dst + TILEB), 16, 0, 0);
      if constexpr (DUAL) {
        __builtin_amdgcn_global_load_lds((JVPFA_GLB(const void))(ktp + ok), (JVPFA_LDS(void))(uintptr_t)(dst + 2 * TILEB), 16, 0, 0);
        __builtin_amdgcn_global_load_lds((JVPFA_GLB(const void))(vtp + ov), (JVPFA_LDS(void))(uintptr_t)(dst + 3 * TILEB), 16, 0, 0);
      }
    }
  };

  // ---- per-lane LDS read offsets (bytes within a tile)
  // K-type: row 32nb + perm32(r), logical chunk 2kk + g
  uint32_t koff[KK];
  {
    const int x = swz_k<CH>(pr32);
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) koff[kk] = pr32 * ROWB + (((2 * kk + g) ^ x) * 16);
  }
  // V-type (transposing read): lane = 32g + 16a + j; it addresses key row 8g + 4hh + j/4 (+16c) and
  // the 8-byte half (j>>1)&1 of logical chunk 4db + 2a + (j&1); it receives keys 16c+8g+4hh+(0..3)
  // at d = 32db + perm32(16a + j).
  uint32_t voff[DB][2];
  {
    const int a = (lane >> 4) & 1, j = lane & 15;
#pragma unroll
    for (int db = 0; db < DB; ++db) {
#pragma unroll
      for (int hh = 0; hh < 2; ++hh) {
        const int row = 8 * g + 4 * hh + (j >> 2);
        const int ch = (4 * db + 2 * a + (j & 1)) ^ swz_v<CH>(row);
        voff[db][hh] = row * ROWB + ch * 16 + 8 * ((j >> 1) & 1);
      }
    }
  }

  Frag<T> Qf[KK], Qtf[DUAL ? KK : 1];
#pragma unroll
  for (int kk = 0; kk < KK; ++kk) {
    Qf[kk] = ld8<T>(Qg + (size_t)qld * D + 16 * kk + 8 * g);
    if constexpr (DUAL) Qtf[kk] = ld8<T>(Qtg + (size_t)qld * D + 16 * kk + 8 * g);
  }
  // the resident operands live in the accumulation register file from here on
#pragma unroll
  for (int kk = 0; kk < KK; ++kk) {
    pin_acc(Qf[kk]);
    if constexpr (DUAL) pin_acc(Qtf[kk]);
  }

  f32x16 Oacc[DB], Tacc[DUAL ? DB : 1];
#pragma unroll
  for (int db = 0; db < DB; ++db) {
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      Oacc[db][e] = 0.f;
      if constexpr (DUAL) Tacc[db][e] = 0.f;
    }
    if constexpr (DUAL) {
      pin_acc(Oacc[db]);
      pin_acc(Tacc[db]);
    }
  }
  float m_i = NEG_INF, l_i = 0.f, mu_i = 0.f;
  // The tangent accumulators work with S' - c_i, c_i a per-row reference close to the row's mu:
  // O' = (P (S' - mu)) V + P V' does not change when a row constant is taken off S', but the 16-bit
  // operand P (S' - c) of the matrix product is rounded in proportion to |S' - c|, and where one key
  // holds most of a row's weight that rounding error is the same multiple of V's row in every column
  // of O', which the backward's row statistic rowsum(gT O') then adds up instead of averaging out.
  // c_i follows the running mu: it is moved to it whenever a half tile brings over four times the weight of
  // everything before it (so always on the first one, and whenever a key arrives that dominates its row),
  // which for ordinary inputs happens on the first tile only; the accumulators are moved along
  // (T -= shift O, mu_acc -= shift l).
  float c_i = 0.f;

  const float sl2 = pr.scale * LOG2E;
  const int64_t mrow = MASK != MASK_NONE ? z * pr.ms[0] + h * pr.ms[1] + (int64_t)qld * pr.ms[2] : 0;
  const uint32_t drop_row = DROP ? drop_row_word(pr, zh, qld) : 0u;  // dropout: this lane's query row, see params.hpp
  bool mask_al = false;  // mask rows can be fetched with aligned vector loads
  if constexpr (MASK != MASK_NONE) mask_al = mask_rows_aligned<T, MASK>(pr);

  int kend = Lk;
  // padded batches: the caller's hint says the mask hides every key from klimit[z] on, so those tiles
  // need not be visited (at least one tile is, which keeps rows without any key well defined)
  if constexpr (MASK != MASK_NONE) {
    if (pr.klimit) kend = min(Lk, max(pr.klimit[z], 1));
  }
  if (pr.causal) kend = min(Lk, q0 + Cfg::BM);
  // Tiles visited: 0 .. ceil(kend/BN)-1, or the caller's list of the tiles of this query block that
  // hold an attended entry (ascending; fully masked tiles contribute exact zeros, so leaving them
  // out changes nothing).  tile_at(i) is the i-th tile visited.
  const int *tlist = nullptr;
  if constexpr (MASK != MASK_NONE) {
    if (pr.tiles_q) tlist = pr.tiles_q + tile_list_offset_q(pr, z, h, qb);
  }
  const int tmax = (Lk + BN - 1) / BN - 1;  // index of the last tile of the sequence: bounds whatever a list holds
  const int ntiles = tlist ? min(max(tlist[0], 1), tmax + 1) : (kend + BN - 1) / BN;
  // List elements are requested a tile ahead, unconditionally (from a harmless address when there is
  // no list: a branch around the read would split the tile loop's straight-line body).
  auto list_slot = [&](int i) { return tlist ? tlist + 1 + i : reinterpret_cast<const int *>(p.q); };

  // The loads of the next tile are not issued in one burst (the vector-memory queue would back up
  // and stall this wave for longer than a whole GEMM phase) but one instruction at a time, spread
  // over the steps of the current tile's matrix products.
  constexpr int NLOAD = IPW * Cfg::NTILE;      // direct-load instructions per wave per tile
  constexpr int NSTEP = 2 * (KK + 2 * DB);     // S and PV steps of the two half tiles
  int ld_rows = 0;
  uint32_t ld_dst = 0;
  const char *ld_p[4] = {nullptr, nullptr, nullptr, nullptr};
  // Past the last tile the loads are pointed at tile 0 again (never read) instead of being
  // predicated off, which keeps every step of the tile loop one straight-line block.
  auto prepare_loads = [&](int stage, int j0, bool on) {
    j0 = on ? j0 : 0;
    ld_rows = Lk - 1 - j0;  // rows past the end re-read the last row; their scores are masked
    ld_dst = lds0 + stage * Cfg::STAGEB + (wave * IPW) * 1024;
    const size_t tb = (size_t)j0 * ROWB;
    ld_p[0] = reinterpret_cast<const char *>(Kg) + tb;
    ld_p[1] = reinterpret_cast<const char *>(Vg) + tb;
    if constexpr (DUAL) {
      ld_p[2] = reinterpret_cast<const char *>(Ktg) + tb;
      ld_p[3] = reinterpret_cast<const char *>(Vtg) + tb;
    }
  };
  auto load_piece = [&](auto pc) {
    constexpr int pi = decltype(pc)::value, i = pi / Cfg::NTILE, ts = pi % Cfg::NTILE;
    const uint32_t off = min(ld_row[i], ld_rows) * ROWB + ((ts & 1) ? ld_cv[i] : ld_ck[i]);
    __builtin_amdgcn_global_load_lds((JVPFA_GLB(const void))(ld_p[ts] + off),
                                     (JVPFA_LDS(void))(uintptr_t)(ld_dst + i * 1024 + ts * TILEB), 16, 0, 0);
  };
  // pieces [ceil(g*NLOAD/NSTEP), ceil((g+1)*NLOAD/NSTEP)) belong to step g
  auto load_step = [&](auto gc) {
    constexpr int g = decltype(gc)::value;
    constexpr int lo = (g * NLOAD + NSTEP - 1) / NSTEP, hi = ((g + 1) * NLOAD + NSTEP - 1) / NSTEP;
    static_for<hi - lo>([&](auto dc) { load_piece(std::integral_constant<int, lo + decltype(dc)::value>{}); });
  };

  // Half-tile body: the 32 keys HB*32 .. HB*32+31 of the tile staged at LDS byte address sbase
  // (layout [K | V | K' | V']); jh is the index of its first key.
  //
  // LDS fragment reads are issued two steps ahead of the matrix products that consume them (a ring
  // of three fragment buffers), through inline asm so that their order and the waits are exactly
  // the ones written here.
  //
  // Rescaling is lazy: the reference point m_i of the exponentials only moves when some row's new
  // maximum exceeds it by more than RESCALE_TAU (log2 units), so p <= 2^TAU and the accumulators,
  // which live in the matrix-core accumulation registers, are touched by VALU code only on the few
  // tiles where the running maximum really grows.  O = acc / l is unchanged by the choice of m_i.
  // (fp16: p multiplies S' - c in a 16-bit operand that overflows at 65504, so the slack is 2^4 there: |S' - c| up
  // to 4 000, where the reference's p <= 1 gives 65 504, see fwd_kernel_v3.hpp; bf16 has the exponent range for 2^8)
  constexpr float RESCALE_TAU = __is_same(T, _Float16) ? 4.f : 8.f;
  constexpr float RESCALE_LEAD = __is_same(T, _Float16) ? 2.f : 0.f;  // the reference point moves this far past the new maximum
  MaskAhead<T, MASK> mcur[2][2], mnext[2][2];  // mask values of this tile and the next: [half tile][16-key group]
  const int klim = min(pr.causal ? qrow : 0x7fffffff, Lk - 1);  // keys above this index are masked
  // EDGE: the half tile may cross the causal diagonal or the end of the sequence, the scale may be
  // negative, or the mask rows are not aligned for vector fetches
  auto half_tile = [&](auto HBc, auto EDGEc, uint32_t sbase, int jh) {
    constexpr int HB = decltype(HBc)::value;
    constexpr bool EDGE = decltype(EDGEc)::value;
    constexpr int KO = HB * 32 * ROWB;  // K at +0, K' at +2*TILEB, V at +TILEB, V' at +3*TILEB
    constexpr int NRS = DUAL ? 2 : 1;   // LDS reads per S step
    constexpr int NRV = DUAL ? 4 : 2;   // LDS reads per PV step
    constexpr int NPV = 2 * DB;         // PV steps: (16-key chunk c, d-block db)

    constexpr int RD = MASK != MASK_NONE ? 4 : 5;  // fragment ring slots (reads run RD-1 steps ahead); the masked kernels need the registers
    constexpr int PD = RD - 1;
    u32x4 ka[RD], kb[RD];
    auto issue_k = [&](auto kkc) {
      constexpr int kk = decltype(kkc)::value;
      const uint32_t ad = sbase + koff[kk];
      ka[kk % RD] = lds_b128<KO>(ad);
      if constexpr (DUAL) kb[kk % RD] = lds_b128<KO + 2 * TILEB>(ad);
    };
    u32x2 va[RD][2], vb[RD][2];
    auto issue_v = [&](auto ic) {
      constexpr int i = decltype(ic)::value, c = i / DB, db = i % DB;
      constexpr int VO = TILEB + (HB * 32 + c * 16) * ROWB;
      const uint32_t a0 = sbase + voff[db][0], a1 = sbase + voff[db][1];
      va[i % RD][0] = lds_tr64<VO>(a0);
      va[i % RD][1] = lds_tr64<VO>(a1);
      if constexpr (DUAL) {
        vb[i % RD][0] = lds_tr64<VO + 2 * TILEB>(a0);
        vb[i % RD][1] = lds_tr64<VO + 2 * TILEB>(a1);
      }
    };

    // score tiles in ordinary vector registers, written by matrix instructions whose B operand (Q, Q')
    // is resident in the accumulation register file
    f32x16 S, Sp;
    // mask values of this half tile: fetched a whole tile earlier (see tile() below)
    MaskAhead<T, MASK> mah[2];
    if constexpr (MASK != MASK_NONE) {
      mah[0] = mcur[HB][0];
      mah[1] = mcur[HB][1];
    }
    static_for<(PD < KK ? PD : KK)>([&](auto kkc) { issue_k(kkc); });
    static_for<KK>([&](auto kkc) {
      constexpr int kk = decltype(kkc)::value;
      constexpr int younger = (KK - 1 - kk < PD - 1) ? KK - 1 - kk : PD - 1;  // read groups issued after this one
      if constexpr (DUAL) lds_wait<younger * NRS>(ka[kk % RD], kb[kk % RD]);
      else lds_wait<younger * NRS>(ka[kk % RD]);
      if constexpr (kk + PD < KK) issue_k(std::integral_constant<int, kk + PD>{});
      load_step(std::integral_constant<int, HB * (KK + NPV) + kk>{});
      const Frag<T> a = __builtin_bit_cast(Frag<T>, ka[kk % RD]);
      if constexpr (DUAL) mma_vra<kk == 0>(Sp, a, Qtf[kk]);
      mma_vra<kk == 0>(S, a, Qf[kk]);
      if constexpr (DUAL) mma_vra<false>(Sp, __builtin_bit_cast(Frag<T>, kb[kk % RD]), Qf[kk]);
    });
    if constexpr (DUAL) tiles_ready(S, Sp);
    else tiles_ready(S);
    float mx;
    constexpr bool general = MASK != MASK_NONE || EDGE;
    if constexpr (general) {
      mx = NEG_INF;
#pragma unroll
      for (int hf = 0; hf < 2; ++hf) {
        const int key0 = jh + 16 * hf + 8 * g;
        float bias[8];
        bool keep[8];
        if constexpr (MASK != MASK_NONE) {
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            if constexpr (MASK == MASK_ADD) bias[e] = mask_bias_of<T, MASK>(mah[hf], e);
            if constexpr (MASK == MASK_BOOL) keep[e] = mask_keep_of<T, MASK>(mah[hf], e);
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
    } else {
      mx = S[0];
#pragma unroll
      for (int e = 1; e < 16; ++e) mx = fmaxf(mx, S[e]);
      mx = pair_max(mx) * sl2;
    }
    // lazy rescaling, decided per query row (rare); the accumulators follow further down, in the block
    // that also re-centres them
    const bool up = mx > m_i + RESCALE_TAU;
    float alpha = 1.f;
    if (__builtin_expect(__any(up), 0)) {
      float m_new = mx;
      if constexpr (RESCALE_LEAD != 0.f) m_new = mx + RESCALE_LEAD;
      alpha = up ? fast_exp2(m_i - m_new) : 1.f;
      m_i = up ? m_new : m_i;
    }
    // V fragments of the first PV steps travel while the softmax runs
    static_for<(PD < NPV ? PD : NPV)>([&](auto ic) { issue_v(ic); });

    const float m_use = (m_i == NEG_INF) ? 0.f : m_i;
    float rs = 0.f, rmu = 0.f;
    if constexpr (general) {
#pragma unroll
      for (int e = 0; e < 16; ++e) S[e] = fast_exp2(S[e] - m_use);
    } else {
#pragma unroll
      for (int e = 0; e < 16; ++e) S[e] = fast_exp2(__builtin_fmaf(S[e], sl2, -m_use));
    }
#pragma unroll
    for (int e = 0; e < 16; ++e) rs += S[e];
    // rare: some row's reference point moved, or (dual) this half tile outweighs what came before it four times
    if (__builtin_expect(__any(up || (DUAL && rs > 4.f * l_i)), 0)) {
      // (the accumulations of the previous half tile finished long ago, behind this half tile's score products;
      // the wait keeps that true wherever the compiler places this block)
      asm volatile("s_nop 15\n\ts_nop 15");
      float neg_shift = 0.f;
      if constexpr (DUAL) {
        const bool outweighs = rs > 4.f * l_i * alpha;
        // both lanes of a query column must decide alike
        const bool move = rare_pair_max(outweighs ? 1.f : 0.f) > 0.f;
        float rc = 0.f;  // rowsum of P (S' - c) over this half tile, old reference
#pragma unroll
        for (int e = 0; e < 16; ++e) rc += S[e] * __builtin_fmaf(Sp[e], pr.scale, -c_i);
        const float tot_l = rare_pair_sum(__builtin_fmaf(l_i, alpha, rs)), tot_mu = rare_pair_sum(__builtin_fmaf(mu_i, alpha, rc));
        const float shift = (move && tot_l > 0.f) ? tot_mu / tot_l : 0.f;
        neg_shift = -shift;
        c_i += shift;
        mu_i = alpha * __builtin_fmaf(neg_shift, l_i, mu_i);
      }
      l_i *= alpha;
#pragma unroll
      for (int db = 0; db < DB; ++db) {
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          if constexpr (DUAL) acc_move_in_place(Tacc[db][e], Oacc[db][e], alpha, neg_shift);
          else Oacc[db][e] = acc_scale(Oacc[db][e], alpha);
        }
      }
    }
    if constexpr (DUAL) {
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const float ps = S[e] * __builtin_fmaf(Sp[e], pr.scale, -c_i);
        Sp[e] = ps;
        rmu += ps;
      }
    }
    l_i += rs;
    if constexpr (DUAL) mu_i += rmu;
    if constexpr (DROP) {  // register e holds key jh + 16(e/8) + 8g + e%8 of this lane's query
      const uint32_t xb = drop_row + (uint32_t)(jh + 8 * g) * DROP_C_KEY;
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
    // the conversions are done (and two issue slots have passed) before the first in-place product reads them
    if constexpr (DUAL) asm volatile("s_nop 1" : "+v"(pf[0]), "+v"(pf[1]), "+v"(psf[0]), "+v"(psf[1]));
    static_for<NPV>([&](auto ic) {
      constexpr int i = decltype(ic)::value, c = i / DB, db = i % DB, sl = i % RD;
      constexpr int younger = (NPV - 1 - i < PD - 1) ? NPV - 1 - i : PD - 1;
      if constexpr (DUAL) lds_wait<younger * NRV>(va[sl][0], va[sl][1], vb[sl][0], vb[sl][1]);
      else lds_wait<younger * NRV>(va[sl][0], va[sl][1]);
      if constexpr (i + PD < NPV) issue_v(std::integral_constant<int, i + PD>{});
      load_step(std::integral_constant<int, HB * (KK + NPV) + KK + i>{});
      const u32x4 av = {va[sl][0][0], va[sl][0][1], va[sl][1][0], va[sl][1][1]};
      const Frag<T> a = __builtin_bit_cast(Frag<T>, av);
      if constexpr (DUAL) {
        // in place (see mfma_acc), and no two consecutive products on the same tile
        const u32x4 bv = {vb[sl][0][0], vb[sl][0][1], vb[sl][1][0], vb[sl][1][1]};
        mfma_acc(Tacc[db], a, psf[c]);
        mfma_acc(Oacc[db], a, pf[c]);
        mfma_acc(Tacc[db], __builtin_bit_cast(Frag<T>, bv), pf[c]);
      } else {
        mma(Oacc[db], a, pf[c]);
      }
    });
  };

  // Mask values travel from HBM or the far caches, further than one phase of matrix products hides:
  // those of tile t+1 are requested at the top of tile t.  [half tile][16-key group] of a tile.
  auto fetch_masks = [&](int tn) {
    if constexpr (MASK != MASK_NONE) {
      const int jn = tn * BN;
      if (mask_al && jn + BN <= Lk) {  // aligned rows, all 64 keys exist: one vector load per 8 keys
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
  issue_loads(0, tcur * BN);
  auto tile = [&](int t, auto EDGEc) {
    const int j0 = tcur * BN;
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
    prepare_loads(stage ^ 1, tnext * BN, t + 1 < ntiles);
    const uint32_t sbase = lds0 + stage * Cfg::STAGEB;
    half_tile(std::integral_constant<int, 0>{}, EDGEc, sbase, j0);
    // always both halves: a half past the last key is fully masked and contributes exact zeros, and a
    // branch here would make the accumulators change register file around it
    half_tile(std::integral_constant<int, 1>{}, EDGEc, sbase, j0 + 32);
    if constexpr (MASK != MASK_NONE) {
      const int listed = list_take(tahead);
      tnext2 = tlist ? min(max(listed, 0), tmax) : tnext2;
    }
    tcur = tnext;
    tnext = tnext2;
  };
  // Tiles that need the general treatment are the last ones; they get a loop of their own so that the
  // common tile carries no limit tests.  (q0 is a multiple of the tile size.)
  int t_edge = Lk / BN;
  if (pr.causal) t_edge = min(t_edge, q0 / BN);
  if (!(sl2 > 0.f) || (MASK != MASK_NONE && !mask_al)) t_edge = 0;
  int t = 0;
  for (; t < ntiles && tcur < t_edge; ++t) tile(t, std::false_type{});
  for (; t < ntiles; ++t) tile(t, std::true_type{});

  // ---- epilogue ---------------------------------------------------------------------------------
  if constexpr (DUAL) accs_ready(Oacc, Tacc);  // the last in-place accumulation has written its registers
  l_i += xor32(l_i);
  if constexpr (DUAL) mu_i += xor32(mu_i);
  const bool dead = !(l_i > 0.f);
  const float inv = dead ? 0.f : 1.f / l_i;
  const float mu_n = mu_i * inv;  // rowsum(P (S' - c)) = mu - c
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
      if constexpr (DUAL) p.mu[(size_t)zh * L + qrow] = dead ? 0.f : mu_n + c_i;
    }
  }
}

}  // namespace jvpfa
