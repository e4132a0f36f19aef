// Software-pipelined fused dual forward for 16-bit element types at D = 128 (and the forward without tangents
// at D = 256): causal, boolean and additive masks (with the key limit and the tile lists), ragged sequence ends, dropout.  Same tiles,
// swizzles, fragment layouts and mathematics as fwd_kernel_v2.hpp; what changes is the order of work
// inside a wave.
//
// A wave issues instructions in order, but a matrix instruction occupies the issue port for a
// fraction of the time the matrix pipe needs to execute it, so independent vector instructions
// placed between two matrix instructions run for free.  The unit of work here is a *slot*, one per
// 32-key half tile h, whose instruction stream interleaves three independent pieces:
//     matrix:  S(h+1) = K Q^T, S'(h+1)            (scores of the next half tile)
//     matrix:  O, T += V^T P(h-1), ...            (accumulation of the previous half tile)
//     vector:  softmax of half tile h             (S(h), S'(h) -> P(h), P(h)S'(h), row sums)
// The vector work is cut into small units and one unit is placed after each matrix instruction.
// K tiles are consumed one slot earlier than V tiles, so the K half and the V half of an LDS stage
// hold different tiles: at the top of iteration t (one workgroup barrier), K(t) and V(t-1) have
// landed and the loads of K(t+1) and V(t) are started.
#pragma once
#include "fwd_kernel_v2.hpp"

namespace jvpfa {

// matrix instructions in program order: score tile in vector registers (B operand resident in the
// accumulation file), and output accumulators in the accumulation file
template <bool FIRST> __device__ __forceinline__ void mfma_s(f32x16 &c, const bf16x8 &a, const bf16x8 &b) {
  if constexpr (FIRST) asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(c) : "v"(a), "a"(b));
  else asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "a"(b));
}
template <bool FIRST> __device__ __forceinline__ void mfma_s(f32x16 &c, const f16x8 &a, const f16x8 &b) {
  if constexpr (FIRST) asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, 0" : "=&v"(c) : "v"(a), "a"(b));
  else asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "a"(b));
}
__device__ __forceinline__ void anchor(const float &x) { asm volatile("" : : "v"(x)); }
__device__ __forceinline__ void anchor(const bf16x8 &x) { asm volatile("" : : "v"(x)); }
__device__ __forceinline__ void anchor(const f16x8 &x) { asm volatile("" : : "v"(x)); }

template <int N>
__device__ __forceinline__ void lds_wait6(u32x4 &a, u32x4 &b, u32x2 &c, u32x2 &d, u32x2 &e, u32x2 &f) {
  asm volatile("s_waitcnt lgkmcnt(%6)" : "+v"(a), "+v"(b), "+v"(c), "+v"(d), "+v"(e), "+v"(f) : "n"(N));
}
template <int N> __device__ __forceinline__ void lds_wait3(u32x4 &a, u32x2 &c, u32x2 &d) {
  asm volatile("s_waitcnt lgkmcnt(%3)" : "+v"(a), "+v"(c), "+v"(d) : "n"(N));
}

// MASK: mask values are requested with vector loads a whole iteration before the softmax that applies them
// (mask.hpp), and tiles that the caller's key limit or tile list leaves out are not visited.
// DROP: dropout on the probabilities (see fwd_kernel.hpp): what enters the products with V, V' is
// P * keep / (1 - p), hashed per entry in the gaps between the matrix instructions; l, mu stay those of the
// full softmax.
// WGS: workgroups meant to share a compute unit.  Without tangents at D = 128, Q and the accumulator are 96
// registers and a stage pair 64 KB, so two fit; the unmasked kernel stays within 256 registers by itself, the
// masked ones are told to.
template <typename T, int D, bool DUAL, int MASK = MASK_NONE, bool DROP = false,
          int WGS = (!DUAL && D <= 128 && (MASK != MASK_NONE || DROP)) ? 2 : 1>
__global__ __launch_bounds__(256, WGS) void fwd3_kernel(const FwdParams p) {
#if defined(__HIP_DEVICE_COMPILE__)  // the host pass only needs the launch stub (and has no buffer descriptor type)
  using Cfg = Fwd2Cfg<T, D, DUAL>;
  constexpr int BN = Cfg::BN, CH = Cfg::CH, ROWB = Cfg::ROWB, TILEB = Cfg::TILEB, IPW = Cfg::IPW;
  constexpr int KK = D / 16, DB = D / 32;
  constexpr int NSS = KK;  // super-steps of a slot: one contraction step of the scores + one (chunk, d-block) of PV
  static_assert(2 * DB == KK, "a slot pairs score step kk with accumulation step kk");
  constexpr float NEG_INF = -__builtin_inff();

  extern __shared__ __attribute__((aligned(1024))) unsigned char smem_raw[];
  // stage s: [K | V | K' | V'] each TILEB bytes; the K-type and V-type halves hold different tiles
  const uint32_t lds0 = (uint32_t)(uintptr_t)smem_raw;

  const Problem &pr = p.pr;
  const int L = pr.L;
  const int nqb = (L + Cfg::BM - 1) / Cfg::BM;
  // small grids: the key tiles of a query block are split over pr.chunks workgroups (see split.hpp)
  const int chunks = pr.chunks;
  const int chunk = chunks > 1 ? (int)(blockIdx.x % chunks) : 0;
  const int id = xcd_remap(chunks > 1 ? blockIdx.x / chunks : blockIdx.x, nqb, pr.Z * pr.H);
  const int zh = id / nqb;
  const int qb = pr.causal ? nqb - 1 - id % nqb : id % nqb;

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid / WAVE), lane = tid % WAVE;
  const int r = lane % 32, g = lane / 32;
  const int pr32 = perm32(r);

  const size_t head = (size_t)zh * L * D;
  // keys: Lk of them, in head h / (H / Hk) of the key/value tensors (L and h themselves for the
  // shapes the reference admits)
  const int q0 = qb * Cfg::BM;
  const int qrow = q0 + wave * 32 + r;
  const int qld = qrow < L ? qrow : L - 1;
  // This workgroup's keys: all of them, or the tiles of its chunk.  From here on key indices are counted from
  // the chunk's first key k0: Lk is the number of keys left from there, and the causal limits move with it.
  int kend = pr.causal ? min(pr.Lk, q0 + Cfg::BM) : pr.Lk;
  // padded batches: the caller's hint says the mask hides every key from klimit[z] on, so those tiles
  // need not be visited (at least one tile is, which keeps rows without any key well defined)
  if constexpr (MASK != MASK_NONE) {
    if (pr.klimit) kend = min(kend, max(__builtin_amdgcn_readfirstlane(pr.klimit[zh / pr.H]), 1));
  }
  const int nt_all = (kend + BN - 1) / BN;
  const int t_first = chunks > 1 ? min(chunk * pr.chunk_tiles, nt_all) : 0;
  // Tiles visited: t_first .. t_first + ntiles - 1, or (with a mask) the caller's list of the tiles of this query
  // block that hold an attended entry (ascending; a tile left out would have contributed exact zeros).
  const int *tlist = nullptr;
  if constexpr (MASK != MASK_NONE) {
    if (pr.tiles_q) tlist = pr.tiles_q + tile_list_offset_q(pr, zh / pr.H, zh % pr.H, qb);
  }
  const int tmax = (pr.Lk + BN - 1) / BN - 1;  // index of the last tile of the sequence: bounds whatever a list holds
  // (what is read from a list is the same in every lane; saying so keeps the tile pointers in scalar registers)
  const int ntiles = tlist ? __builtin_amdgcn_readfirstlane(min(max(tlist[0], 1), tmax + 1))
                           : (chunks > 1 ? min(nt_all - t_first, pr.chunk_tiles) : nt_all);  // 0: nothing for this chunk
  const int k0 = t_first * BN;
  const int Lk = pr.Lk - k0;
  // partial results of a chunk: [chunk][row][O | T][D] floats, then [chunk][row][m, l, mu_acc, c]
  const size_t nrows = (size_t)pr.Z * pr.H * L, prow = (size_t)chunk * nrows + (size_t)zh * L + qrow;
  float *part_stat = pr.part + (size_t)chunks * nrows * 2 * D + prow * 4;
  if (chunks > 1 && ntiles <= 0) {  // no tile falls to this chunk (short causal rows): it weighs nothing
    if (qrow < L && g == 0) {
      const f32x4 none = {-__builtin_inff(), 0.f, 0.f, 0.f};
      *reinterpret_cast<f32x4 *>(part_stat) = none;
    }
    return;
  }
  const size_t kvhead = (((size_t)(zh / pr.H) * pr.Hk + (zh % pr.H) / (pr.H / pr.Hk)) * pr.Lk + k0) * D;
  const T *Qg = reinterpret_cast<const T *>(p.q) + head;
  const char *Kg = reinterpret_cast<const char *>(reinterpret_cast<const T *>(p.k) + kvhead);
  const char *Vg = reinterpret_cast<const char *>(reinterpret_cast<const T *>(p.v) + kvhead);
  const T *Qtg = DUAL ? reinterpret_cast<const T *>(p.qt) + head : nullptr;
  const char *Ktg = DUAL ? reinterpret_cast<const char *>(reinterpret_cast<const T *>(p.kt) + kvhead) : nullptr;
  const char *Vtg = DUAL ? reinterpret_cast<const char *>(reinterpret_cast<const T *>(p.vt) + kvhead) : nullptr;

  // ---- direct loads (see fwd_kernel_v2.hpp): instruction i of this wave fills chunks 64*(wave*IPW+i)..+63
  int ld_row[IPW];
  uint32_t ld_ck[IPW], ld_cv[IPW];
#pragma unroll
  for (int i = 0; i < IPW; ++i) {
    const int lc = 64 * (wave * IPW + i) + lane;
    const int row = lc / CH, cp = lc % CH;
    ld_row[i] = row;
    ld_ck[i] = (cp ^ swz_k<CH>(row)) * 16;
    ld_cv[i] = (cp ^ swz_v<CH>(row)) * 16;
  }
  uint32_t koff[KK];
  {
    const int x = swz_k<CH>(pr32);
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) koff[kk] = pr32 * ROWB + (((2 * kk + g) ^ x) * 16);
  }
  // (the second transposing read of a fragment takes rows 4 further down: the same chunk, since the V-type swizzle
  // only looks at the two low bits of the row, so it is the first one's address plus a constant)
  uint32_t voff[DB];
  {
    const int a = (lane >> 4) & 1, j = lane & 15;
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      const int row = 8 * g + (j >> 2);
      const int ch = (4 * db + 2 * a + (j & 1)) ^ swz_v<CH>(row);
      voff[db] = row * ROWB + ch * 16 + 8 * ((j >> 1) & 1);
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

  f32x16 Oacc[DB], Tacc[DUAL ? DB : 1];
#pragma unroll
  for (int db = 0; db < DB; ++db) {
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      Oacc[db][e] = 0.f;
      if constexpr (DUAL) Tacc[db][e] = 0.f;
    }
    pin_acc(Oacc[db]);
    if constexpr (DUAL) pin_acc(Tacc[db]);
  }
  float m_i = NEG_INF, l_i = 0.f, mu_i = 0.f;
  float c_i = 0.f;  // per-row reference taken off S' (see fwd_kernel_v2.hpp): follows the running mu

  const float sl2 = pr.scale * LOG2E;
  const bool neg_scale = !(sl2 > 0.f);
  const int qlim = pr.causal ? qrow - k0 : 0x7fffffff;  // keys above this index are masked
  const int64_t mrow = MASK != MASK_NONE ? (zh / pr.H) * pr.ms[0] + (zh % pr.H) * pr.ms[1] + (int64_t)qld * pr.ms[2] : 0;
  bool mask_al = false;  // mask rows can be fetched with aligned vector loads
  if constexpr (MASK != MASK_NONE) mask_al = mask_rows_aligned<T, MASK>(pr);
  const uint32_t drop_row = DROP ? drop_row_word(pr, zh, qld) : 0u;  // dropout: this lane's query row, see params.hpp
  // List elements are requested an iteration ahead, unconditionally (from a harmless address when there is no
  // list: a branch around the read would split the loop's straight-line body).
  auto list_slot = [&](int i) { return tlist ? tlist + 1 + i : reinterpret_cast<const int *>(p.q); };
  auto tile_first_key = [&](int i) {  // first key of the i-th tile visited (i clamped to the last one)
    const int ic = min(i, max(ntiles - 1, 0));
    return (tlist ? min(max(tlist[1 + ic], 0), tmax) : ic) * BN;
  };

  // ---- next-tile loads, one instruction per super-step -------------------------------------------
  constexpr int NLOAD = IPW * Cfg::NTILE;
  // the loads of an iteration are spread over its first NSTEP super-steps, not all 2*NSS of them: the
  // last load then has half a slot to land before the barrier that waits for it
  constexpr int NSTEP = 3 * NSS / 2;
  uint32_t ld_dst_k = 0, ld_dst_v = 0;
  // Buffer loads: the descriptor of a tensor holds (start of the tile, bytes left in the head) and the
  // per-lane offset is a constant of the kernel, so a load needs no vector arithmetic; rows past the
  // end of the sequence, and tiles that do not exist, are out of range and read as zeros.
  __amdgpu_buffer_rsrc_t ld_rs[4];
  uint32_t ldo_k[IPW], ldo_v[IPW];
#pragma unroll
  for (int i = 0; i < IPW; ++i) {
    ldo_k[i] = ld_row[i] * ROWB + ld_ck[i];
    ldo_v[i] = ld_row[i] * ROWB + ld_cv[i];
  }
  auto tile_rsrc = [&](const char *base, int j, bool exists) {
    const int rows = exists ? max(Lk - j, 0) : 0;
    return __builtin_amdgcn_make_buffer_rsrc((void *)(base + (size_t)j * ROWB), 0, rows * ROWB, 0x00020000);
  };
  // iteration t loads K(t+1) into the K half of stage (t+1)&1 and V(t) into the V half of stage t&1
  // (jv, jk: first keys of tile t and of tile t + 1)
  auto prepare_loads = [&](int t, int jv, int jk) {
    if constexpr (MASK != MASK_NONE) {  // (the same in every lane, see above)
      jv = __builtin_amdgcn_readfirstlane(jv);
      jk = __builtin_amdgcn_readfirstlane(jk);
    }
    ld_dst_k = lds0 + ((t + 1) & 1) * Cfg::STAGEB + (wave * IPW) * 1024;
    ld_dst_v = lds0 + (t & 1) * Cfg::STAGEB + (wave * IPW) * 1024;
    ld_rs[0] = tile_rsrc(Kg, jk, t + 1 < ntiles);
    ld_rs[1] = tile_rsrc(Vg, jv, t < ntiles);
    if constexpr (DUAL) {
      ld_rs[2] = tile_rsrc(Ktg, jk, t + 1 < ntiles);
      ld_rs[3] = tile_rsrc(Vtg, jv, t < ntiles);
    }
  };
  auto prepare_first = [&](int jk) {
    ld_dst_k = lds0 + (wave * IPW) * 1024;
    ld_rs[0] = tile_rsrc(Kg, jk, true);
    if constexpr (DUAL) ld_rs[2] = tile_rsrc(Ktg, jk, true);
  };
  auto load_piece = [&](auto pc) {
    constexpr int pi = decltype(pc)::value, i = pi / Cfg::NTILE, ts = pi % Cfg::NTILE;
    constexpr bool vt = (ts & 1) != 0;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(ld_rs[ts], (JVPFA_LDS(void))(uintptr_t)((vt ? ld_dst_v : ld_dst_k) + i * 1024 + ts * TILEB),
                                             16, vt ? ldo_v[i] : ldo_k[i], 0, 0, 0);
  };
  auto load_step = [&](auto gc) {
    constexpr int gi = decltype(gc)::value;
    if constexpr (gi < NSTEP) {
      constexpr int lo = (gi * NLOAD + NSTEP - 1) / NSTEP, hi = ((gi + 1) * NLOAD + NSTEP - 1) / NSTEP;
      static_for<hi - lo>([&](auto dc) { load_piece(std::integral_constant<int, lo + decltype(dc)::value>{}); });
    }
  };

  // fp16: p <= 2^TAU multiplies S' - c in a 16-bit operand that overflows at 65504, so the slack is 2^4 there
  // (|S' - c| up to 4 000; the reference's p <= 1 gives 65 504).  The running maximum of a row of unit-variance
  // logits grows by about 2 log2 units between its first tile and its 64th, so 2^4 is still rarely crossed; with
  // 2^2 every row crosses it about once and the rescale block costs 27 % of the kernel.  bf16 has the exponent
  // range for 2^8.
  constexpr float RESCALE_TAU = __is_same(T, _Float16) ? 4.f : 8.f;
  // ... and when the reference point does move, fp16 puts it 2 log2 units above the new maximum (p <= 1/4 on that
  // tile, and the next move waits for a maximum 6 above this one), so that the smaller slack does not make the
  // moves frequent: rows whose maximum climbs by more than 4 over the sequence are common, by more than 6 rare
  constexpr float RESCALE_LEAD = __is_same(T, _Float16) ? 2.f : 0.f;
  constexpr int NQ = DUAL ? 3 : 1, NP = DUAL ? 3 : 1;  // matrix instructions per super-step: scores, accumulation
  constexpr int NRS = DUAL ? 2 : 1, NRV = DUAL ? 4 : 2;  // LDS reads per super-step
  constexpr int NU = 38;                                 // vector units of one softmax
  constexpr int NU0 = 5;                                 // ... of which this many form its front
  constexpr int RD = 4, PD = RD - 1;           // fragment ring slots; reads run PD super-steps ahead

  // One slot.  QK: scores of a half tile (K rows at LDS address kaddr) into Sn, Spn.  PV: accumulate
  // the half tile whose V rows are at vaddr, with fragments pfp, psfp.  SM: softmax of Sc, Spc (first
  // key jh) into pfn, psfn.  GEN: 0 the softmax takes the scores as they are; 1 it adds the mask terms madd
  // (0 or -inf for a boolean mask, the bias in log2 units for an additive one) to the scaled scores; 2 it
  // applies the causal / sequence-end limits (kernels without a mask).  With a mask, a slot that forms scores
  // also forms the mask terms that go with them, in its gaps: madd is read by the front of the softmax and
  // refilled behind it from the mask words mah of the half tile whose scores the slot forms (keys
  // 16 c + 8 g .. + 7 in mah[c]; keys past the end come masked from the fetch).
  // LB: index of the first load step of this slot, or -1.
  u32x4 ka[RD], kb[RD];
  u32x2 va[RD][2], vb[RD][2];
  auto slot = [&](auto QKc, auto PVc, auto SMc, auto GENc, auto LBc, auto PREc, auto NEXTc, uint32_t kaddr, uint32_t vaddr, f32x16 &Sc,
                  f32x16 &Spc, f32x16 &Sn, f32x16 &Spn, Frag<T>(&pfp)[2], Frag<T>(&psfp)[2], Frag<T>(&pfn)[2],
                  Frag<T>(&psfn)[2], int jh, const MaskAhead<T, MASK>(&mah)[2], float (&madd)[16]) {
    constexpr bool QK = decltype(QKc)::value, PV = decltype(PVc)::value, SM = decltype(SMc)::value;
    constexpr int GENL = decltype(GENc)::value;
    constexpr bool GEN = GENL != 0, LIM = GENL == 2;
    static_assert(MASK == MASK_NONE ? GENL != 1 : (GENL == 1 || !SM), "a masked softmax adds its mask terms, no other does");
    constexpr bool PREC = MASK != MASK_NONE && QK;  // mask terms for the scores this slot forms
    constexpr int NPRE = PREC ? 8 : 0;              // ... as this many vector units of two entries
    uint32_t vzero = 0u, vninf = 0xff800000u;
    if constexpr (PREC && MASK == MASK_BOOL) asm volatile("" : "+v"(vzero), "+v"(vninf));  // vector registers that hold 0 and -inf
    // dropout: register e holds key jh + 16(e/8) + 8g + e%8 of this lane's query
    const uint32_t xb = DROP ? drop_row + (uint32_t)(jh + 8 * g) * DROP_C_KEY : 0u;
    constexpr int LB = decltype(LBc)::value;
    // PRE: the reads of the first PD super-steps were issued by the previous slot; NEXT: issue those of
    // the next slot, which works on the other half of the same two tiles
    constexpr bool PRE = decltype(PREc)::value, NEXT = decltype(NEXTc)::value;
    constexpr int MPS = (QK ? NQ : 0) + (PV ? NP : 0);  // matrix instructions per super-step
    constexpr int NG = NSS * MPS;                       // gaps of the slot
    constexpr int NUS = SM ? NU - NU0 : 0;                  // softmax units behind the front
    constexpr int UPG = (NUS + NPRE + NG - 1) / NG;         // vector units per gap
    constexpr int RPS = (QK ? NRS : 0) + (PV ? NRV : 0);
    static_assert((PD - 1) * RPS <= 15, "lgkmcnt is a 4-bit counter");
    static_assert(!NEXT || (NSS % RD == 0 && QK && PV), "the fragment ring continues into the next slot");

    // ---- softmax state and units ----------------------------------------------------------------
    float mxa = NEG_INF, mxb = NEG_INF, mx = NEG_INF, alpha = 1.f, m_use = 0.f, rs = 0.f, rmu = 0.f, xarg = 0.f;
    float pv[16], sv[16];
    bool any_up = false, outweighs = false, up_l = false;
    auto unit = [&](auto uc) {
      constexpr int u = decltype(uc)::value;
      if constexpr (u == 0 || u == 1) {  // row maximum over registers 8u .. 8u+7
        float m8 = NEG_INF;
#pragma unroll
        for (int e = 8 * u; e < 8 * u + 8; ++e) {
          if constexpr (GEN) {
            const int key = jh + 16 * (e / 8) + 8 * g + (e % 8);
            float s = MASK != MASK_NONE ? __builtin_fmaf(Sc[e], sl2, madd[e]) : Sc[e] * sl2;
            if constexpr (LIM) {
              s = (key <= qlim) ? s : NEG_INF;
              s = (key < Lk) ? s : NEG_INF;
            }
            Sc[e] = s;
            m8 = fmaxf(m8, s);
          } else {
            m8 = (e == 8 * u) ? Sc[e] : fmaxf(m8, Sc[e]);
          }
        }
        if constexpr (u == 0) mxa = m8;
        else mxb = m8;
        anchor(m8);
      } else if constexpr (u == 2) {
        mx = pair_max(fmaxf(mxa, mxb));
        if constexpr (!GEN) mx *= sl2;
        anchor(mx);
      } else if constexpr (u == 3) {
        // lazy rescale, decided per query row: the reference point only moves when the row maximum
        // exceeds it by more than RESCALE_TAU (log2 units)
        const bool up = mx > m_i + RESCALE_TAU;
        up_l = up;
        if constexpr (!DUAL) any_up = __any(up);
        float m_new = mx;
        if constexpr (RESCALE_LEAD != 0.f) m_new = mx + RESCALE_LEAD;
        alpha = up ? fast_exp2(m_i - m_new) : 1.f;
        m_i = up ? m_new : m_i;
        anchor(alpha);
      } else if constexpr (u == 4) {
        m_use = (m_i == NEG_INF) ? 0.f : m_i;
        xarg = GEN ? Sc[0] - m_use : __builtin_fmaf(Sc[0], sl2, -m_use);
      } else if constexpr (u < 37) {
        constexpr int e = (u - 5) / 2;
        if constexpr ((u - 5) % 2 == 0) {
          // the exponent of the next element is formed behind this element's exponential, so that a vector
          // instruction stands between a transcendental and the first reader of its result (in the next gap)
          pv[e] = fast_exp2(xarg);
          if constexpr (e + 1 < 16) xarg = GEN ? Sc[e + 1] - m_use : __builtin_fmaf(Sc[e + 1], sl2, -m_use);
          if constexpr (DUAL) sv[e] = __builtin_fmaf(Spc[e], pr.scale, -c_i);
          anchor(pv[e]);
        } else {
          rs += pv[e];
          if constexpr (DUAL) {
            sv[e] *= pv[e];
            rmu += sv[e];
          }
          if constexpr (DROP) {  // the row sums above are those of the full softmax; 1 / (1 - p) waits for the epilogue
            const bool kept = drop_finish(xb + (uint32_t)(16 * (e / 8) + (e % 8)) * DROP_C_KEY) >= pr.drop_thr;
            pv[e] = kept ? pv[e] : 0.f;
            if constexpr (DUAL) sv[e] = kept ? sv[e] : 0.f;
          }
          if constexpr (e % 2 == 1) {
            constexpr int c = e / 8, j = e % 8;
            pfn[c][j - 1] = (T)pv[e - 1];
            pfn[c][j] = (T)pv[e];
            if constexpr (DUAL) {
              psfn[c][j - 1] = (T)sv[e - 1];
              psfn[c][j] = (T)sv[e];
            }
            if constexpr (j == 7) {
              anchor(pfn[c]);
              if constexpr (DUAL) anchor(psfn[c]);
            }
          }
          anchor(rs);
        }
      } else {
        l_i = __builtin_fmaf(l_i, alpha, rs);
        if constexpr (DUAL) {
          mu_i = __builtin_fmaf(mu_i, alpha, rmu);
          // this half tile holds over 4/5 of the row's weight so far: the reference of S' follows (rare)
          outweighs = 1.25f * rs > l_i;
          any_up = __any(up_l | outweighs);  // one test for both rare events (no branch inside the slot)
        }
      }
    };
    // (anchor(): an empty asm statement that consumes a value; it keeps the unit that produced the value
    // at its place in the instruction stream, between the matrix instructions written around it)
    // the vector work that follows matrix instruction number gi of the slot
    auto gap = [&](auto gc) {
      constexpr int gi = decltype(gc)::value;
      static_for<UPG>([&](auto uc) {
        constexpr int k = gi * UPG + decltype(uc)::value;
        if constexpr (k < NUS) {
          unit(std::integral_constant<int, NU0 + k>{});
        } else if constexpr (k < NUS + NPRE) {  // mask terms of entries 2 (k - NUS), + 1 for the next softmax
          static_for<2>([&](auto jc) {
            constexpr int e = 2 * (k - NUS) + decltype(jc)::value;
            if constexpr (MASK == MASK_BOOL) {  // byte e % 8 of the eight
              const uint32_t word = (e % 8) < 4 ? (uint32_t)mah[e / 8].w : (uint32_t)(mah[e / 8].w >> 32);
              madd[e] = mask_term_of_byte<e % 4>(word, vzero, vninf);
            }
            if constexpr (MASK == MASK_ADD) madd[e] = (float)mah[e / 8].f[e % 8] * LOG2E;
          });
          anchor(madd[2 * (k - NUS)]);
          anchor(madd[2 * (k - NUS) + 1]);
        }
      });
      __builtin_amdgcn_sched_barrier(0);
    };

    // ---- fragment reads --------------------------------------------------------------------------
    // step NSS + j is step j of the next slot (rows 32 further down in the same tiles)
    auto issue = [&](auto ic) {
      constexpr int i = decltype(ic)::value % NSS, sl = i % RD;
      constexpr int HO = (decltype(ic)::value / NSS) * 32 * ROWB;
      if constexpr (QK) {
        const uint32_t ad = kaddr + koff[i];
        ka[sl] = lds_b128<HO>(ad);
        if constexpr (DUAL) kb[sl] = lds_b128<HO + 2 * TILEB>(ad);
      }
      if constexpr (PV) {
        constexpr int c = i / DB, db = i % DB;
        constexpr int VO = HO + TILEB + c * 16 * ROWB;
        const uint32_t a0 = vaddr + voff[db];
        static_assert(VO + (DUAL ? 2 * TILEB : 0) + 4 * ROWB < 65536, "the offset field of an LDS instruction has 16 bits");
        va[sl][0] = lds_tr64<VO>(a0);
        va[sl][1] = lds_tr64<VO + 4 * ROWB>(a0);
        if constexpr (DUAL) {
          vb[sl][0] = lds_tr64<VO + 2 * TILEB>(a0);
          vb[sl][1] = lds_tr64<VO + 2 * TILEB + 4 * ROWB>(a0);
        }
      }
    };

    if constexpr (SM) {
      if constexpr (DUAL) tiles_ready(Sc, Spc);
      else tiles_ready(Sc);
    }
    if constexpr (!PRE) static_for<(PD < NSS ? PD : NSS)>([&](auto ic) { issue(ic); });
    // the front of the softmax (row maximum, reference point) runs while the first fragments travel
    if constexpr (SM) static_for<NU0>([&](auto uc) { unit(uc); });
    static_for<NSS>([&](auto ic) {
      constexpr int i = decltype(ic)::value, sl = i % RD;
      constexpr int younger = (NEXT ? PD - 1 : ((NSS - 1 - i < PD - 1) ? NSS - 1 - i : PD - 1)) * RPS;
      if constexpr (QK && PV) {
        if constexpr (DUAL) lds_wait6<younger>(ka[sl], kb[sl], va[sl][0], va[sl][1], vb[sl][0], vb[sl][1]);
        else lds_wait3<younger>(ka[sl], va[sl][0], va[sl][1]);
      } else if constexpr (QK) {
        if constexpr (DUAL) lds_wait<younger>(ka[sl], kb[sl]);
        else lds_wait<younger>(ka[sl]);
      } else {
        if constexpr (DUAL) lds_wait<younger>(va[sl][0], va[sl][1], vb[sl][0], vb[sl][1]);
        else lds_wait<younger>(va[sl][0], va[sl][1]);
      }
      if constexpr (i + PD < NSS || NEXT) issue(std::integral_constant<int, i + PD>{});
      if constexpr (LB >= 0) load_step(std::integral_constant<int, (LB >= 0 ? LB : 0) + i>{});
      constexpr int c = i / DB, db = i % DB;
      constexpr int G0 = i * MPS;
      Frag<T> fa, fb, fv, fw;
      if constexpr (QK) {
        fa = __builtin_bit_cast(Frag<T>, ka[sl]);
        if constexpr (DUAL) fb = __builtin_bit_cast(Frag<T>, kb[sl]);
      }
      if constexpr (PV) {
        const u32x4 av = {va[sl][0][0], va[sl][0][1], va[sl][1][0], va[sl][1][1]};
        fv = __builtin_bit_cast(Frag<T>, av);
        if constexpr (DUAL) {
          const u32x4 bv = {vb[sl][0][0], vb[sl][0][1], vb[sl][1][0], vb[sl][1][1]};
          fw = __builtin_bit_cast(Frag<T>, bv);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
      if constexpr (DUAL) {
        // order: no two consecutive matrix instructions update the same tile
        if constexpr (QK && PV) {
          mfma_s<i == 0>(Spn, fa, Qtf[i]);
          gap(std::integral_constant<int, G0 + 0>{});
          mfma_acc(Oacc[db], fv, pfp[c]);
          gap(std::integral_constant<int, G0 + 1>{});
          mfma_s<i == 0>(Sn, fa, Qf[i]);
          gap(std::integral_constant<int, G0 + 2>{});
          mfma_acc(Tacc[db], fv, psfp[c]);
          gap(std::integral_constant<int, G0 + 3>{});
          mfma_s<false>(Spn, fb, Qf[i]);
          gap(std::integral_constant<int, G0 + 4>{});
          mfma_acc(Tacc[db], fw, pfp[c]);
          gap(std::integral_constant<int, G0 + 5>{});
        } else if constexpr (QK) {
          mfma_s<i == 0>(Spn, fa, Qtf[i]);
          gap(std::integral_constant<int, G0 + 0>{});
          mfma_s<i == 0>(Sn, fa, Qf[i]);
          gap(std::integral_constant<int, G0 + 1>{});
          mfma_s<false>(Spn, fb, Qf[i]);
          gap(std::integral_constant<int, G0 + 2>{});
        } else {
          mfma_acc(Tacc[db], fv, psfp[c]);
          gap(std::integral_constant<int, G0 + 0>{});
          mfma_acc(Oacc[db], fv, pfp[c]);
          gap(std::integral_constant<int, G0 + 1>{});
          mfma_acc(Tacc[db], fw, pfp[c]);
          gap(std::integral_constant<int, G0 + 2>{});
        }
      } else {
        if constexpr (QK) {
          mfma_s<i == 0>(Sn, fa, Qf[i]);
          gap(std::integral_constant<int, G0 + 0>{});
        }
        if constexpr (PV) {
          mfma_acc(Oacc[db], fv, pfp[c]);
          gap(std::integral_constant<int, G0 + (QK ? 1 : 0)>{});
        }
      }
    });
    if constexpr (SM) {
      if (any_up) {  // rare: some row's reference point (of S or of S') moved; the accumulators follow it
        asm volatile("s_nop 15\n\ts_nop 15");  // the last accumulation above has written its registers
        float neg_shift = 0.f;
        if constexpr (DUAL) {
          // l_i, mu_i already hold this half tile (with the old reference); both lanes of a query column
          // must decide alike
          const bool move = rare_pair_max(outweighs ? 1.f : 0.f) > 0.f;
          const float tot_l = rare_pair_sum(l_i), tot_mu = rare_pair_sum(mu_i);
          const float shift = (move && tot_l > 0.f) ? tot_mu / tot_l : 0.f;
          neg_shift = -shift;
          c_i += shift;
          mu_i = __builtin_fmaf(neg_shift, l_i, mu_i);
          // the operand P (S' - c) of this half tile again, with the new reference (the exponentials come
          // out exactly as before: same instructions on the same registers)
          float m_again = m_use;
          anchor(m_again);  // a value of its own: otherwise every exponential above is kept alive for this path
#pragma unroll
          for (int e = 0; e < 16; ++e) {
            float pe;
            if constexpr (GEN) pe = fast_exp2(Sc[e] - m_again);
            else pe = fast_exp2(__builtin_fmaf(Sc[e], sl2, -m_again));
            if constexpr (DROP) pe = drop_finish(xb + (uint32_t)(16 * (e / 8) + (e % 8)) * DROP_C_KEY) >= pr.drop_thr ? pe : 0.f;
            psfn[e / 8][e % 8] = (T)(pe * __builtin_fmaf(Spc[e], pr.scale, -c_i));
          }
        }
#pragma unroll
        for (int db = 0; db < DB; ++db) {
#pragma unroll
          for (int e = 0; e < 16; ++e) {
            if constexpr (DUAL) acc_move_in_place(Tacc[db][e], Oacc[db][e], alpha, neg_shift);
            else Oacc[db][e] = acc_scale(Oacc[db][e], alpha);
          }
        }
      }
    }
  };

  using B0 = std::false_type;
  using B1 = std::true_type;
  using XP = std::integral_constant<bool, NSS % RD == 0>;  // fragment prefetch across the two slots of an iteration
  constexpr bool MASKED = MASK != MASK_NONE;
  using GI = std::integral_constant<int, MASKED ? 1 : 0>;  // softmax of interior tiles, see slot()
  using GE = std::integral_constant<int, MASKED ? 1 : 2>;  // ... of tiles that meet a limit (with a mask the fetch applies it)
  f32x16 SX, SpX, SY, SpY;
  Frag<T> pfA[2], psfA[2], pfB[2], psfB[2];

  // Mask words of the two half tiles of an iteration's tile, each by 16-key group, and of the tile after it.
  // They travel from HBM or the far caches: those of iteration t + 1 are requested at the top of iteration t.
  MaskAhead<T, MASK> mcur[2][2], mnext[2][2];
  float madd[16];  // mask terms of the scores in flight, see slot()
  auto fetch_half = [&](MaskAhead<T, MASK>(&dst)[2], int jh) {
    if constexpr (MASKED) {
      if (mask_al && jh + 32 <= pr.Lk) {  // aligned rows, all 32 keys exist: one vector load per 8 keys
#pragma unroll
        for (int c = 0; c < 2; ++c) dst[c] = mask_fetch8<T, MASK>(pr, mrow, jh + 16 * c + 8 * g);
      } else {
#pragma unroll
        for (int c = 0; c < 2; ++c) dst[c] = mask_fetch8_lim<T, MASK>(pr, mrow, jh + 16 * c + 8 * g);
      }
    }
  };
  // first keys of the tiles of iterations t - 1, t, t + 1
  int jA = 0, jB = 0, jC = BN;
  if constexpr (MASKED) {
    jB = __builtin_amdgcn_readfirstlane(tile_first_key(0));
    jC = __builtin_amdgcn_readfirstlane(tile_first_key(1));
  }
  // at the end of iteration t: the tile of iteration t + 2 comes from the list element requested at its top
  auto advance = [&](int t, int tahead) {
    if constexpr (MASKED) {
      const int listed = list_take(tahead);
      jA = jB;
      jB = jC;
      jC = (tlist ? min(max(listed, 0), tmax) : min(t + 2, ntiles - 1)) * BN;
    }
  };

  // ---- prologue: K(0) in one burst ---------------------------------------------------------------
  prepare_first(jB);
  static_for<NLOAD>([&](auto pc) {
    if constexpr (decltype(pc)::value % 2 == 0) load_piece(pc);
  });
  fetch_half(mcur[0], jB);
  fetch_half(mcur[1], jB + 32);
  auto kad = [&](int t, int hb) { return lds0 + (t & 1) * Cfg::STAGEB + hb * 32 * ROWB; };

  // iteration 0: scores of half tiles 0 and 1, softmax of half tile 0
  __builtin_amdgcn_s_waitcnt(0x0F70);
  __syncthreads();
  {
    int tahead = 0;
    if constexpr (MASKED) {
      tahead = list_request(list_slot(min(2, ntiles - 1)));
      fetch_half(mnext[0], jC);
      fetch_half(mnext[1], jC + 32);
    }
    prepare_loads(0, jB, jC);
    slot(B1{}, B0{}, B0{}, GE{}, std::integral_constant<int, 0>{}, B0{}, B0{}, kad(0, 0), 0u, SX, SpX, SY, SpY, pfA, psfA, pfB, psfB, jB,
         mcur[0], madd);
    slot(B1{}, B0{}, B1{}, GE{}, std::integral_constant<int, NSS>{}, B0{}, B0{}, kad(0, 1), 0u, SY, SpY, SX, SpX, pfB, psfB, pfA, psfA, jB,
         mcur[1], madd);
    advance(0, tahead);
  }
  auto iteration = [&](int t, auto GENc) {
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this wave's share of K(t), V(t-1) has landed
    __syncthreads();                      // ... everyone's has, and K(t-1), V(t-2) are no longer read
    int tahead = 0;
    if constexpr (MASKED) {
      tahead = list_request(list_slot(min(t + 2, ntiles - 1)));
#pragma unroll
      for (int i = 0; i < 4; ++i) mcur[i / 2][i % 2] = mnext[i / 2][i % 2];
      fetch_half(mnext[0], jC);
      fetch_half(mnext[1], jC + 32);
    } else {
      jA = (t - 1) * BN;
      jB = t * BN;
      jC = (t + 1) * BN;
    }
    prepare_loads(t, jB, jC);
    slot(B1{}, B1{}, B1{}, GENc, std::integral_constant<int, 0>{}, B0{}, XP{}, kad(t, 0), kad(t - 1, 0), SX, SpX, SY, SpY, pfA, psfA, pfB, psfB,
         jA + 32, mcur[0], madd);
    slot(B1{}, B1{}, B1{}, GENc, std::integral_constant<int, NSS>{}, XP{}, B0{}, kad(t, 1), kad(t - 1, 1), SY, SpY, SX, SpX, pfB, psfB, pfA, psfA,
         jB, mcur[1], madd);
    advance(t, tahead);
  };
  // Without a mask, iterations whose softmax needs the causal / sequence-end limits form the tail of the loop;
  // they get a loop of their own so that the common iteration is one straight-line block.
  int t = 1;
  if constexpr (!MASKED) {
    int t_gen = (Lk >= 32) ? (Lk - 32) / BN + 1 : 0;
    if (pr.causal) t_gen = min(t_gen, max(q0 - k0 + 32, 0) / BN);
    t_gen = neg_scale ? 1 : max(1, t_gen);
    for (; t < min(t_gen, ntiles); ++t) iteration(t, GI{});
  }
  for (; t < ntiles; ++t) iteration(t, GE{});
  // drain: softmax of the last half tile, accumulation of the last two
  __builtin_amdgcn_s_waitcnt(0x0F70);
  __syncthreads();
  if constexpr (!MASKED) jA = (ntiles - 1) * BN;
  slot(B0{}, B1{}, B1{}, GE{}, std::integral_constant<int, -1>{}, B0{}, B0{}, 0u, kad(ntiles - 1, 0), SX, SpX, SY, SpY, pfA, psfA, pfB, psfB,
       jA + 32, mcur[0], madd);
  slot(B0{}, B1{}, B0{}, GE{}, std::integral_constant<int, -1>{}, B0{}, B0{}, 0u, kad(ntiles - 1, 1), SY, SpY, SX, SpX, pfB, psfB, pfA, psfA, 0,
       mcur[0], madd);
  // the last accumulation has written its registers
  if constexpr (DUAL) accs_ready(Oacc, Tacc);
  else accs_ready(Oacc);

  // ---- epilogue ---------------------------------------------------------------------------------
  l_i += xor32(l_i);
  if constexpr (DUAL) mu_i += xor32(mu_i);
  if (chunks > 1) {  // this chunk's share, left as it stands for the merge kernel
    if (qrow < L) {
      float *pa = pr.part + prow * 2 * D;
#pragma unroll
      for (int db = 0; db < DB; ++db) {
#pragma unroll
        for (int hf = 0; hf < 2; ++hf) {
          float o8[8], t8[8];
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            o8[e] = Oacc[db][8 * hf + e];
            if constexpr (DUAL) t8[e] = Tacc[db][8 * hf + e];
          }
          const int d0 = 32 * db + 16 * hf + 8 * g;
          store8<float>(pa + d0, o8);
          if constexpr (DUAL) store8<float>(pa + D + d0, t8);
        }
      }
      if (g == 0) {
        const f32x4 st = {m_i, l_i, mu_i, c_i};
        *reinterpret_cast<f32x4 *>(part_stat) = st;
      }
    }
    return;
  }
  const bool dead = !(l_i > 0.f);
  const float inv_l = dead ? 0.f : 1.f / l_i;
  const float mu_n = mu_i * inv_l;
  const float inv = DROP ? inv_l * pr.drop_rinv : inv_l;  // the kept entries' 1 / (1 - p) is common to O and T
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
      if constexpr (DUAL) p.mu[(size_t)zh * L + qrow] = dead ? 0.f : mu_n + c_i;  // mu_n = rowsum(P (S' - c))
    }
  }
#endif
}

}  // namespace jvpfa
