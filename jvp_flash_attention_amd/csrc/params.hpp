// Kernel-side argument blocks (the C ABI structs of include/jvpfa.h, already validated).
#pragma once
#include <stdint.h>

namespace jvpfa {

// MASK_BITS is a boolean mask read by the dk/dv kernels from its bit-packed transposed copy (Problem::bits_k),
// MASK_TILE an additive mask whose 64-query x 128-key tiles those kernels stream through LDS like the operand
// tiles (rows of 16-byte aligned, contiguous keys); both exist as template arguments of those kernels only.
enum MaskKind { MASK_NONE = 0, MASK_BOOL = 1, MASK_ADD = 2, MASK_BITS = 3, MASK_TILE = 4 };

struct Problem {
  int Z, H, L;  // batch, query heads, query length
  // Key/value length and heads; equal to L and H for the shapes the reference admits
  // (jvp_attention.py:2367-2378).  Query head h reads key/value head h / (H / Hk).
  int Lk, Hk;
  int causal;
  float scale;
  const void *mask;
  int64_t ms[4];  // element strides (z, h, query, key)
  const int *klimit;  // per batch entry: keys at or past this index are masked by the mask (hint), or null
  // Lists of the tiles that hold an attended entry, or null: per mask plane and 128-row block,
  // 1 + ceil(L/64) ints (count >= 1, then ascending indices of 64-wide tiles).  tiles_q: key tiles
  // per query block; tiles_k: query tiles per key block.
  const int *tiles_q, *tiles_k;
  // A boolean mask packed along the query axis, or null: per mask plane, tile of 64 query rows and key a pair
  // of words, bit i of word hf being the mask entry of (query 64 * tile + 32 * hf + i, key); rows past L are
  // zero bits.  The dk/dv kernels, whose lanes own a key, read one pair per 64 queries instead of 64 bytes a
  // mask row apart.
  const uint32_t *bits_k;
  // Split of the streamed tiles of one block of owned rows over `chunks` workgroups (1 = no split), used when
  // a launch would otherwise leave most compute units idle: workgroup c of a block takes the tiles
  // c * chunk_tiles .. (c + 1) * chunk_tiles - 1 and writes fp32 partial results to `part`, which a merge
  // kernel adds up.  Only the kernels for 16-bit element types, D = 128, without a mask.
  int chunks, chunk_tiles;
  float *part;
  // Dropout on the attention probabilities (0 in drop_thr: none).  Entry (z, h, query i, key j) is kept when
  // drop_entry_hash(...) >= drop_thr, and kept entries are scaled by drop_rinv = 1 / (1 - p); the same function of
  // (seed, z, h, i, j) in the forward, both backward kernels and jvpfa_dropout_keep.
  uint32_t drop_thr, drop_s0, drop_s1;
  float drop_rinv;
};

// Counter-based keep decision, shaped so that a kernel pays a handful of vector instructions per entry whichever
// way it walks the matrix.  Query rows are taken in blocks of 32: the block (z H + h) ceil(L / 32) + i / 32 and the
// seed go through a full 64 -> 32 bit mix (once per lane or per tile in a kernel); inside a block the word moves by a
// constant per row and a constant per key (two Weyl sequences), and two multiply-xorshift rounds finish the entry.
constexpr uint32_t DROP_C_KEY = 0x9E3779B1u, DROP_C_ROW = 0x85EBCA77u;
__host__ __device__ inline uint32_t drop_block_hash(uint64_t block, uint32_t s0, uint32_t s1) {
  uint32_t x = ((uint32_t)block * 0x9E3779B1u) ^ s0;
  x ^= (uint32_t)(block >> 32) * 0x85EBCA77u + s1;
  x ^= x >> 16;
  x *= 0x7feb352du;
  x ^= x >> 15;
  x *= 0x846ca68bu;
  x ^= x >> 16;
  return x;
}
__host__ __device__ inline uint32_t drop_finish(uint32_t x) {
  x ^= x >> 16;
  x *= 0x7feb352du;
  x ^= x >> 15;
  x *= 0x846ca68bu;
  return x;
}
// the word of row i of head zh = z H + h before the key's share: drop_finish(drop_row_word + j * DROP_C_KEY) is the hash
__host__ __device__ inline uint32_t drop_row_word(const Problem &pr, int zh, int i) {
  const uint64_t block = (uint64_t)zh * (uint64_t)((pr.L + 31) / 32) + (uint64_t)(i >> 5);
  return drop_block_hash(block, pr.drop_s0, pr.drop_s1) + (uint32_t)(i & 31) * DROP_C_ROW;
}
// 1 / (1 - p) for a kept entry, 0 for a dropped one, from the entry's word
__host__ __device__ inline float drop_scale_of(const Problem &pr, uint32_t word) {
  return drop_finish(word) >= pr.drop_thr ? pr.drop_rinv : 0.f;
}
__host__ __device__ inline float drop_scale(const Problem &pr, int zh, int i, int j) {
  return drop_scale_of(pr, drop_row_word(pr, zh, i) + (uint32_t)j * DROP_C_KEY);
}

constexpr int TILE_BLOCK = 128, TILE_W = 64;  // geometry of the tile lists
// First element of the list of (plane of (z, h), block).  tiles_q: blocks of 128 query rows, each with up to
// ceil(Lk / 64) key tiles; tiles_k: blocks of 128 keys, each with up to ceil(L / 64) query tiles.
__host__ __device__ inline size_t tile_list_plane(const Problem &pr, int z, int h) {
  const int hm = pr.ms[1] ? pr.H : 1;
  return (size_t)(pr.ms[0] ? z : 0) * hm + (pr.ms[1] ? h : 0);
}
__host__ __device__ inline size_t tile_list_offset_q(const Problem &pr, int z, int h, int block) {
  const int nblk = (pr.L + TILE_BLOCK - 1) / TILE_BLOCK, nt = (pr.Lk + TILE_W - 1) / TILE_W;
  return (tile_list_plane(pr, z, h) * nblk + block) * (size_t)(nt + 1);
}
__host__ __device__ inline size_t tile_list_offset_k(const Problem &pr, int z, int h, int block) {
  const int nblk = (pr.Lk + TILE_BLOCK - 1) / TILE_BLOCK, nt = (pr.L + TILE_W - 1) / TILE_W;
  return (tile_list_plane(pr, z, h) * nblk + block) * (size_t)(nt + 1);
}

// first word of the plane of (z, h) in the bit-packed mask
__host__ __device__ inline size_t mask_bits_offset(const Problem &pr, int z, int h) {
  return tile_list_plane(pr, z, h) * (size_t)((pr.L + 63) / 64) * (size_t)pr.Lk * 2;
}

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
