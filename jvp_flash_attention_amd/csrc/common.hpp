// Shared device-side building blocks for the gfx950 JVP flash-attention kernels:
// MFMA fragment types, the 32x32x16 matrix-core step for bf16 / fp16 / fp32, and the
// global->LDS tile movers (row-major and transposed).
//
// Fragment convention (wave64, v_mfma_f32_32x32x16_{bf16,f16}): with r = lane % 32 and
// g = lane / 32, the A operand of lane holds A[row r][k = 8g .. 8g+7], the B operand holds
// B[k = 8g .. 8g+7][col r], and accumulator register e holds C[row 8(e/4) + 4g + e%4][col r].
// Every kernel here loads A rows through perm32(), which swaps bits 2 and 3 of the row index,
// so that accumulator register e of lane-group g belongs to logical row 16(e/8) + 8g + e%8:
// eight consecutive logical rows per half of the register file.  That makes an accumulator tile
// directly reusable as the k-contiguous B (or A) operand of the next matrix product.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace jvpfa {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr float LOG2E = 1.4426950408889634f;
constexpr float LN2 = 0.6931471805599453f;
constexpr int WAVE = 64;

template <typename T> struct VecOf;
template <> struct VecOf<__bf16> { using x8 = bf16x8; using x4 = bf16x4; };
template <> struct VecOf<_Float16> { using x8 = f16x8; using x4 = f16x4; };
template <> struct VecOf<float> { using x8 = f32x8; using x4 = f32x4; };
template <typename T> using Frag = typename VecOf<T>::x8;
template <typename T> using Quad = typename VecOf<T>::x4;

__device__ __forceinline__ int perm32(int i) { return (i & ~12) | ((i & 4) << 1) | ((i & 8) >> 1); }

// One 32x32 accumulator update over 16 values of the contraction index.
__device__ __forceinline__ void mma(f32x16 &c, const bf16x8 &a, const bf16x8 &b) {
  c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ void mma(f32x16 &c, const f16x8 &a, const f16x8 &b) {
  c = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
}
// fp32: eight 32x32x2 steps; step e contracts the two k values {e, 8+e} of the group of 16.
__device__ __forceinline__ void mma(f32x16 &c, const f32x8 &a, const f32x8 &b) {
#pragma unroll
  for (int e = 0; e < 8; ++e) c = __builtin_amdgcn_mfma_f32_32x32x2f32(a[e], b[e], c, 0, 0, 0);
}

// Eight consecutive accumulator registers (one half of a 32x32 tile) as an operand fragment.
template <typename T> __device__ __forceinline__ Frag<T> to_frag(const f32x16 &x, int half) {
  Frag<T> f;
#pragma unroll
  for (int e = 0; e < 8; ++e) f[e] = (T)x[8 * half + e];
  return f;
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float xor32(float x) { return __shfl_xor(x, 32, 64); }
// Combine a value with the one held by the lane 32 away (the other half of a query column):
// v_permlane32_swap of x with itself returns (lower half broadcast, upper half broadcast).
__device__ __forceinline__ float pair_max(float x) {
  auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float pair_sum(float x) {
  auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// Eight consecutive elements from a 16-byte aligned address (LDS or global).
template <typename T> __device__ __forceinline__ Frag<T> ld8(const T *p) {
  return *reinterpret_cast<const Frag<T> *>(p);
}
template <> __device__ __forceinline__ f32x8 ld8<float>(const float *p) {
  f32x4 lo = *reinterpret_cast<const f32x4 *>(p), hi = *reinterpret_cast<const f32x4 *>(p + 4);
  f32x8 f = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
  return f;
}
template <typename T> __device__ __forceinline__ Frag<T> lds_frag(const T *p) { return ld8<T>(p); }

// 16-byte chunk of global memory, or zeros when the row is out of range.
__device__ __forceinline__ u32x4 ld_chunk(const void *p, bool valid) {
  u32x4 z = {0u, 0u, 0u, 0u};
  return valid ? *reinterpret_cast<const u32x4 *>(p) : z;
}

// Row-major tile: dst[row][0..D) <- src[(row0 + row)][0..D) for row < ROWS; rows >= nvalid are zero.
template <typename T, int ROWS, int D, int NT>
__device__ __forceinline__ void copy_rows(T *dst, int ld, const T *src, int nvalid, int tid) {
  constexpr int EPC = 16 / sizeof(T);
  constexpr int CPR = D / EPC;
  constexpr int TOTAL = ROWS * CPR;
#pragma unroll
  for (int it = 0; it < (TOTAL + NT - 1) / NT; ++it) {
    int c = tid + it * NT;
    if (TOTAL % NT == 0 || c < TOTAL) {
      int row = c / CPR, col = (c % CPR) * EPC;
      u32x4 x = ld_chunk(src + (size_t)row * D + col, row < nvalid);
      *reinterpret_cast<u32x4 *>(dst + row * ld + col) = x;
    }
  }
}

// Transposed tile: dst[col][row] <- src[row][col].  A task is 4 rows x one 16-byte chunk of
// columns; its 4x(EPC) block is transposed in registers and written as EPC vectors of 4 rows.
template <typename T, int ROWS, int D, int NT>
__device__ __forceinline__ void copy_rows_transposed(T *dst, int ld, const T *src, int nvalid, int tid) {
  constexpr int EPC = 16 / sizeof(T);
  constexpr int CPR = D / EPC;
  constexpr int RG = ROWS / 4;
  constexpr int TOTAL = RG * CPR;
#pragma unroll
  for (int it = 0; it < (TOTAL + NT - 1) / NT; ++it) {
    int c = tid + it * NT;
    if (TOTAL % NT == 0 || c < TOTAL) {
      int rg = c % RG, cc = c / RG;
      union { u32x4 v; T e[EPC]; } in[4];
#pragma unroll
      for (int i = 0; i < 4; ++i)
        in[i].v = ld_chunk(src + (size_t)(4 * rg + i) * D + cc * EPC, 4 * rg + i < nvalid);
#pragma unroll
      for (int e = 0; e < EPC; ++e) {
        Quad<T> o;
#pragma unroll
        for (int i = 0; i < 4; ++i) o[i] = in[i].e[e];
        *reinterpret_cast<Quad<T> *>(dst + (cc * EPC + e) * ld + 4 * rg) = o;
      }
    }
  }
}

// The two movers above cut in two, so that the global loads of the next tile travel while the
// current tile is computed: fetch_* issues the loads into registers, put_* (after the compute, behind
// a barrier) writes them to LDS.
template <typename T, int ROWS, int D, int NT> struct RowChunks {
  static constexpr int EPC = 16 / sizeof(T), CPR = D / EPC, TOTAL = ROWS * CPR, N = (TOTAL + NT - 1) / NT;
  u32x4 x[N];
};
template <typename T, int ROWS, int D, int NT>
__device__ __forceinline__ void fetch_rows(RowChunks<T, ROWS, D, NT> &r, const T *src, int nvalid, int tid) {
  using R = RowChunks<T, ROWS, D, NT>;
#pragma unroll
  for (int it = 0; it < R::N; ++it) {
    const int c = tid + it * NT;
    if (R::TOTAL % NT == 0 || c < R::TOTAL) {
      const int row = c / R::CPR, col = (c % R::CPR) * R::EPC;
      r.x[it] = ld_chunk(src + (size_t)row * D + col, row < nvalid);
    }
  }
}
template <typename T, int ROWS, int D, int NT>
__device__ __forceinline__ void put_rows(T *dst, int ld, const RowChunks<T, ROWS, D, NT> &r, int tid) {
  using R = RowChunks<T, ROWS, D, NT>;
#pragma unroll
  for (int it = 0; it < R::N; ++it) {
    const int c = tid + it * NT;
    if (R::TOTAL % NT == 0 || c < R::TOTAL) {
      const int row = c / R::CPR, col = (c % R::CPR) * R::EPC;
      *reinterpret_cast<u32x4 *>(dst + row * ld + col) = r.x[it];
    }
  }
}
// tasks of 4 rows x one 16-byte chunk of columns; one fetch serves a transposed put and, where a
// tile is needed both ways, a row-major put as well
template <typename T, int ROWS, int D, int NT> struct QuadChunks {
  static constexpr int EPC = 16 / sizeof(T), CPR = D / EPC, RG = ROWS / 4, TOTAL = RG * CPR, N = (TOTAL + NT - 1) / NT;
  u32x4 x[N][4];
};
template <typename T, int ROWS, int D, int NT>
__device__ __forceinline__ void fetch_quads(QuadChunks<T, ROWS, D, NT> &r, const T *src, int nvalid, int tid) {
  using R = QuadChunks<T, ROWS, D, NT>;
#pragma unroll
  for (int it = 0; it < R::N; ++it) {
    const int c = tid + it * NT;
    if (R::TOTAL % NT == 0 || c < R::TOTAL) {
      const int rg = c % R::RG, cc = c / R::RG;
#pragma unroll
      for (int i = 0; i < 4; ++i)
        r.x[it][i] = ld_chunk(src + (size_t)(4 * rg + i) * D + cc * R::EPC, 4 * rg + i < nvalid);
    }
  }
}
template <typename T, int ROWS, int D, int NT>
__device__ __forceinline__ void put_quads_transposed(T *dst, int ld, const QuadChunks<T, ROWS, D, NT> &r, int tid) {
  using R = QuadChunks<T, ROWS, D, NT>;
#pragma unroll
  for (int it = 0; it < R::N; ++it) {
    const int c = tid + it * NT;
    if (R::TOTAL % NT == 0 || c < R::TOTAL) {
      const int rg = c % R::RG, cc = c / R::RG;
      union { u32x4 v; T e[R::EPC]; } in[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) in[i].v = r.x[it][i];
#pragma unroll
      for (int e = 0; e < R::EPC; ++e) {
        Quad<T> o;
#pragma unroll
        for (int i = 0; i < 4; ++i) o[i] = in[i].e[e];
        *reinterpret_cast<Quad<T> *>(dst + (cc * R::EPC + e) * ld + 4 * rg) = o;
      }
    }
  }
}
template <typename T, int ROWS, int D, int NT>
__device__ __forceinline__ void put_quads_rows(T *dst, int ld, const QuadChunks<T, ROWS, D, NT> &r, int tid) {
  using R = QuadChunks<T, ROWS, D, NT>;
#pragma unroll
  for (int it = 0; it < R::N; ++it) {
    const int c = tid + it * NT;
    if (R::TOTAL % NT == 0 || c < R::TOTAL) {
      const int rg = c % R::RG, cc = c / R::RG;
#pragma unroll
      for (int i = 0; i < 4; ++i) *reinterpret_cast<u32x4 *>(dst + (4 * rg + i) * ld + cc * R::EPC) = r.x[it][i];
    }
  }
}

// Blocks are dealt round-robin to the 8 XCDs (each with its own L2).  Re-deal them so that the blocks
// of one head (which share its K/V) land on one XCD and are worked on there at about the same time:
// XCD x takes heads x, x+8, x+16, ... one after another.  Dealing heads round-robin rather than in
// contiguous ranges matters when the work per head varies with the batch entry (padded batches): every
// XCD then gets its share of every batch entry.  Returns head * per_head + block.
__device__ __forceinline__ int xcd_remap(int bid, int per_head, int heads) {
  constexpr int NXCD = 8;
  const int total = per_head * heads;
  if (heads % NXCD == 0) {
    const int x = bid % NXCD, j = bid / NXCD;  // j: arrival order within XCD x
    return ((j / per_head) * NXCD + x) * per_head + j % per_head;
  }
  if (total % NXCD != 0) return bid;
  return (bid % NXCD) * (total / NXCD) + bid / NXCD;  // contiguous ranges of blocks
}

// Store 8 consecutive elements of type T converted from fp32.
template <typename T> __device__ __forceinline__ void store8(T *dst, const float *x) {
  Frag<T> f;
#pragma unroll
  for (int e = 0; e < 8; ++e) f[e] = (T)x[e];
  *reinterpret_cast<Frag<T> *>(dst) = f;
}
template <> __device__ __forceinline__ void store8<float>(float *dst, const float *x) {
  f32x4 lo = {x[0], x[1], x[2], x[3]}, hi = {x[4], x[5], x[6], x[7]};
  *reinterpret_cast<f32x4 *>(dst) = lo;
  *reinterpret_cast<f32x4 *>(dst + 4) = hi;
}

}  // namespace jvpfa
