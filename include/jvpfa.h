/*
 * jvpfa.h -- C ABI of the MI355X (gfx950) JVP flash-attention kernels.
 *
 * Plain pointers and sizes only; no torch types.  Every entry point is
 * stateless, launches asynchronously on the HIP stream it is given, owns no
 * memory and allocates none: the caller passes every input, output and
 * workspace buffer as a device pointer.  Return value: 0 on success, a
 * negative JVPFA_E_* code otherwise (jvpfa_error_string() names it).  Safe to
 * call from any thread; two calls that write the same buffers race.
 *
 * Tensors q, k, v, their tangents, outputs and gradients are dense row-major
 * (Z, H, L, D) (k, v and what belongs to them: (Z, Hk, Lk, D) when a call says so); row statistics are fp32 (Z, H, L).  The mask, when present,
 * is addressed with four element strides (0 = broadcast along that axis), so
 * a key-padding mask of shape [Z,1,1,L] is read in place.
 *
 * Each function names the part of the reference
 * (jvp_flash_attention/jvp_attention.py, "JA") whose device work it replaces.
 */
#ifndef JVPFA_H
#define JVPFA_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define JVPFA_ABI_VERSION 8

enum jvpfa_dtype { JVPFA_BF16 = 0, JVPFA_FP16 = 1, JVPFA_FP32 = 2 };

/* JA:2429-2446 classifies masks as 0 none / 1 boolean / 2 additive float. */
enum jvpfa_mask_kind { JVPFA_MASK_NONE = 0, JVPFA_MASK_BOOL = 1, JVPFA_MASK_ADD = 2 };

enum jvpfa_status {
  JVPFA_OK = 0,
  JVPFA_E_NULL = -1,      /* a required pointer is NULL */
  JVPFA_E_SHAPE = -2,     /* Z,H,L < 1, D not in {32, 64, 128, 256}, dropout_p outside [0, 1) */
  JVPFA_E_DTYPE = -3,     /* dtype / mask_kind out of range */
  JVPFA_E_ALIGN = -4,     /* a tensor pointer is not 16-byte aligned */
  JVPFA_E_CONFLICT = -5,  /* causal together with a mask (JA:2380-2381 raises ValueError) */
  JVPFA_E_LAUNCH = -6,    /* hipGetLastError() reported a launch failure */
  JVPFA_E_ABI = -7,       /* struct_size is not this library's: caller built from another header */
  JVPFA_E_SCRATCH = -8    /* jvpfa_bwd_static: Z*H*L is more than jvpfa_bwd_static_max_rows() */
};

/* Shape, numeric type and masking shared by forward and backward. */
typedef struct jvpfa_problem {
  int32_t Z, H, L, D; /* D in {32, 64, 128, 256}; the reference also admits 16 (JA:2371-2374): a caller pads
                       * q, k, v (and tangents, gradients) with zero columns to 32 and drops them from the results */
  int32_t dtype;      /* enum jvpfa_dtype: element type of q,k,v,o and their tangents/gradients */
  int32_t causal;     /* 0/1; lower-triangular (query index >= key index), JA:253-258 */
  int32_t mask_kind;  /* enum jvpfa_mask_kind */
  float sm_scale;     /* logits = sm_scale * q.k (+ additive mask); JA:2395-2396 default D^-0.5 */
  const void *mask;   /* bool: uint8, nonzero = attend (JA:241-245); additive: same dtype as q,
                         added to the scaled logits (SDPA semantics) */
  int64_t mask_stride[4]; /* element strides over (z, h, query, key); 0 broadcasts */
  /* Dropout on the attention probabilities: 0 <= dropout_p < 1, 0 = none.  Entry (z, h, query, key) is kept or
   * dropped by a counter-based hash of (dropout_seed, z, h, query, key) and kept entries are scaled by 1/(1 - p), as
   * torch's scaled_dot_product_attention does; forward and backward of one call pair must get the same seed.
   * jvpfa_dropout_keep() writes the keep pattern out.  The reference carries dead code for dropout and raises
   * NotImplementedError (JA:94-122, JA:271-277, JA:2356-2357).  Costs bf16 / fp16 calls 6 - 13 % at D = 128
   * (a third where the unmasked, non-causal forward leaves its software-pipelined kernel), about 30 % at D = 64,
   * fp32 1 - 6 %.
   * The seed is an argument of the kernels: a launch recorded into a HIP graph replays with the seed it was
   * recorded with, i.e. the same keep pattern on every replay; a caller that wants a fresh pattern per step
   * records the graph anew (or runs the dropout calls outside it). */
  float dropout_p;
  uint64_t dropout_seed;
} jvpfa_problem;

/*
 * Fused dual forward.  Replaces the device work of JA:662-1033 (_attn_fwd) with
 * its inner loop JA:125-336, launched from JVPAttn.forward (JA:2592-2631).
 * With qt = kt = vt = NULL it is the plain forward (ENABLE_JVP False, JA:2365)
 * and ot / mu may be NULL.
 *   o  = softmax(S) v
 *   ot = (P * (S' - mu)) v + P vt,   S' = sm_scale (qt k^T + q kt^T)
 *   M  = log2-domain log-sum-exp of S per query row (JA:1017-1022); +inf for a row
 *        with every key masked (such rows give o = ot = 0, JA:1011-1015)
 *   mu = rowsum(P * S'), saved for the backward (the reference does not keep it)
 */
typedef struct jvpfa_fwd_args {
  uint32_t struct_size; /* sizeof(jvpfa_fwd_args) */
  jvpfa_problem p;
  const void *q, *k, *v;
  const void *qt, *kt, *vt; /* all three NULL, or all three set */
  void *o, *ot;
  float *M, *mu;
  /* optional hint for padded batches, Z int32 values on the device or NULL.  The caller promises
   * that the mask itself masks every key index >= key_limit[z] for all heads and queries of batch
   * z; key tiles past the limit are then skipped instead of read and masked.  No counterpart in the
   * reference, which reads the full (Z,H,L,L) mask (JA:2383-2388).  Ignored without a mask. */
  const int32_t *key_limit;
  /* optional lists of the key tiles that hold an attended entry, written by jvpfa_mask_tiles() for
   * this same mask (and the same Lk), or NULL.  Tiles not listed are skipped instead of read and masked.
   * When set, key_limit is ignored.  Ignored without a mask. */
  const int32_t *tiles_q;
  /* shape of k, v, kt, vt when it is not q's -- Lk keys (any length >= 1) and Hk key/value heads, Hk a divisor
   * of p.H; query head h reads key/value head h / (H / Hk).  0 means "as q" (p.L, p.H).  k, v and
   * their tangents are then (Z, Hk, Lk, D), the mask strides address (z, h, query, key) with Lk keys,
   * and causal means key index <= query index.  The reference requires q, k, v of one shape
     * (JA:2367-2378).  key_limit then counts the Lk keys; the tile lists must have been made for the same Lk
   * (any Hk: they belong to the mask planes, which follow the query heads). */
  int32_t Lk, Hk;
  /* optional workspace for small grids, or NULL: jvpfa_fwd_split_workspace_bytes(&p, Lk) bytes of device memory,
   * 16-byte aligned, contents don't-care.  When a launch would have fewer workgroups than the GPU has compute
   * units (one long sequence, few heads), the key tiles of every query block are then split over up to 8
   * workgroups that leave fp32 partial results there, and a second kernel merges them into o, ot, M, mu
   * (bf16 / fp16, D = 128, no mask; ignored otherwise).  Results agree with the unsplit launch to rounding.
   * No counterpart in the reference (one program per 32 query rows whatever the grid, JA:2474-2476). */
  void *split_workspace;
  uint64_t split_workspace_bytes;
} jvpfa_fwd_args;

int jvpfa_fwd(const jvpfa_fwd_args *args, void *hip_stream);

/* Bytes of split_workspace with which jvpfa_fwd would split this problem on the current device; 0 if it would
 * not (grid large enough, or a kernel that does not split). */
size_t jvpfa_fwd_split_workspace_bytes(const jvpfa_problem *p, int32_t Lk);

/*
 * Backward of  Loss = <go, o> + <gt, ot>.  Replaces the device work of
 * _attn_bwd_preprocess (JA:1384-1411), _attn_bwd / _attn_bwd_causal
 * (JA:2008-2233, JA:1710-2005) with their inner loops JA:1415-1707, launched
 * from JVPAttn.backward (JA:2921-2974), and adds the gradient through the
 * tangent output, which the reference lacks (JA:2831 ignores its second
 * incoming gradient).
 *   gt == NULL            first-order backward: needs q,k,v,o,M,go -> dq,dk,dv
 *                         (tangent pointers and ot, mu may be NULL)
 *   gt != NULL            needs all of q,k,v,qt,kt,vt,o,ot,M,mu; go may be NULL (= 0)
 *   dqt,dkt,dvt           optional outputs (all NULL or all set; need gt != NULL):
 *                         gradients w.r.t. the tangent inputs
 * workspace: jvpfa_bwd_workspace_bytes(Z,H,L) bytes of device memory, 16-byte
 * aligned, contents don't-care on entry (row statistics of the pre-pass).
 */
typedef struct jvpfa_bwd_args {
  uint32_t struct_size; /* sizeof(jvpfa_bwd_args) */
  jvpfa_problem p;
  const void *q, *k, *v;
  const void *qt, *kt, *vt;
  const void *o, *ot;
  const float *M, *mu;
  const void *go, *gt;
  void *dq, *dk, *dv;
  void *dqt, *dkt, *dvt;
  void *workspace;
  const int32_t *key_limit; /* as in jvpfa_fwd_args */
  const int32_t *tiles_q;   /* as in jvpfa_fwd_args (used by the dq kernels) */
  const int32_t *tiles_k;   /* the other list of jvpfa_mask_tiles() (dk/dv kernels);
                               tiles_q and tiles_k are both NULL or both set */
  int32_t Lk, Hk;           /* as in jvpfa_fwd_args; dk, dv, dkt, dvt have the shape of k */
  const uint32_t *mask_bits; /* optional, boolean masks only: the copy written by jvpfa_mask_bits(), or NULL */
} jvpfa_bwd_args;

int jvpfa_bwd(const jvpfa_bwd_args *args, void *hip_stream);

size_t jvpfa_bwd_workspace_bytes(int32_t Z, int32_t H, int32_t L);

/*
 * jvpfa_bwd for callers that cannot hand over a workspace because they cannot allocate one: code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  No counterpart in
 * the reference (whose backward allocates its `delta` with torch, JA:2883).  Same arguments and
 * results as jvpfa_bwd; args->workspace is ignored, the row statistics of the pre-pass live in an
 * array inside the library instead: 3 * JVPFA_STATIC_ROWS floats (12 MiB) of device memory per GPU
 * the library runs on, held until the process ends.  The call allocates nothing and frees nothing.
 * Limit: Z*H*L (rounded up to a multiple of 4) <= JVPFA_STATIC_ROWS, otherwise JVPFA_E_SCRATCH and
 * nothing is launched.  The GPU the stream belongs to must be the current device.  Every call on a
 * GPU uses that GPU's one array: two calls that overlap in time on one GPU (different streams, or
 * different threads) race; calls on one stream, one after another, are fine.
 * The first call on a GPU looks the array's address up (hipGetSymbolAddress, which makes the runtime load
 * the library's code object there and commit the 12 MiB): make that one call, with any valid arguments,
 * outside graph capture and before memory is measured; every later call on that GPU only launches kernels.
 */
#define JVPFA_STATIC_ROWS (1 << 20)
int jvpfa_bwd_static(const jvpfa_bwd_args *args, void *hip_stream);
size_t jvpfa_bwd_static_max_rows(void);

/*
 * Tile lists of a mask: which 64-wide tiles hold at least one attended entry (boolean: nonzero;
 * additive: anything but -inf).  The kernels then visit only those; a mask that is block-diagonal,
 * banded or padded on both axes costs time in proportion to its attended area.  No counterpart in
 * the reference, which visits every tile of the materialised (Z,H,L,L) mask (JA:2383-2388).
 *   tiles_q  for every mask plane and block of 128 query rows: the 64-key tiles to visit
 *   tiles_k  for every mask plane and block of 128 keys: the 64-query tiles to visit
 * Either may be NULL (not both): the forward needs tiles_q only.
 * A mask plane is a (z, h) pair, with one plane along an axis whose mask stride is 0.  The mask has p->L query
 * rows and Lk keys (0 = as p->L).  A list of tiles_q is 1 + ceil(Lk/64) int32 values, one of tiles_k
 * 1 + ceil(L/64): the count (at least 1), then the tile indices in ascending order.  The buffers are
 * jvpfa_mask_tiles_bytes(p, Lk, 0) and jvpfa_mask_tiles_bytes(p, Lk, 1) bytes of device memory, 4-byte
 * aligned.  The lists describe the mask's contents: rebuild them when those change.  Only p->Z, H, L, dtype,
 * mask_kind, mask and mask_stride are read.  Every element type and head dim walks them (kernels with 32-wide
 * tiles take a listed tile as two).
 */
size_t jvpfa_mask_tiles_bytes(const jvpfa_problem *p, int32_t Lk, int32_t keys_owned);
int jvpfa_mask_tiles(const jvpfa_problem *p, int32_t Lk, int32_t *tiles_q, int32_t *tiles_k, void *hip_stream);

/*
 * A boolean mask packed along the query axis, for the dk/dv kernels: their lanes own a key and walk down the
 * queries, so from the mask itself they fetch one byte per entry, a mask row apart; from this copy one pair of
 * 32-bit words per 64 queries.  No counterpart in the reference, whose kernels load the mask block by block
 * (JA:1451-1463, JA:1607-1619).  Layout: for every mask plane (as for jvpfa_mask_tiles), tile of 64 query
 * rows t < ceil(L/64), key j < Lk and half hf < 2 the word [((plane * ceil(L/64) + t) * Lk + j) * 2 + hf], whose
 * bit i is 1 where the mask entry of (query 64 t + 32 hf + i, key j) is nonzero; bits of rows past L are 0.  The
 * buffer is jvpfa_mask_bits_bytes(p, Lk) bytes of device memory (an eighth of the broadcast mask), 8-byte aligned; it
 * describes the mask's contents: rebuild it when those change.  Only p->Z, H, L, mask_kind (must be
 * JVPFA_MASK_BOOL), mask and mask_stride are read.  Handing it to jvpfa_bwd is optional and changes no result;
 * the kernels for 16-bit element types at D <= 128 use it, the others read the mask itself.
 */
size_t jvpfa_mask_bits_bytes(const jvpfa_problem *p, int32_t Lk);
int jvpfa_mask_bits(const jvpfa_problem *p, int32_t Lk, uint32_t *bits, void *hip_stream);

/*
 * The keep pattern of dropout for this problem (only Z, H, L, dropout_p, dropout_seed are read) and Lk keys
 * (0 = as L): keep[z][h][query][key] = 1 for a kept entry, 0 for a dropped one, Z*H*L*Lk bytes of device memory.
 * For tests and for callers that want to reproduce a call with another implementation.
 */
int jvpfa_dropout_keep(const jvpfa_problem *p, int32_t Lk, uint8_t *keep, void *hip_stream);

/* JVPFA_ABI_VERSION of the loaded library. */
int jvpfa_abi_version(void);

/* Static, NUL-terminated description of a jvpfa_status value. */
const char *jvpfa_error_string(int status);

#ifdef __cplusplus
}
#endif
#endif /* JVPFA_H */
