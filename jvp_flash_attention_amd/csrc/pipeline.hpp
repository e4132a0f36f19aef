// Building blocks of the gfx950 memory pipeline shared by the forward and backward kernels for
// 16-bit element types: direct-to-LDS tile loads, XOR chunk swizzles, LDS fragment reads whose
// issue points and waits are fixed by the program text, and in-place accumulator scaling.
#pragma once
#include <utility>

#include "common.hpp"

namespace jvpfa {

#define JVPFA_LDS(T) __attribute__((address_space(3))) T *
#define JVPFA_GLB(T) __attribute__((address_space(1))) T *

typedef short s16x4 __attribute__((ext_vector_type(4)));

template <int... Is, typename F>
__device__ __forceinline__ void static_for_impl(std::integer_sequence<int, Is...>, F &&f) {
  (f(std::integral_constant<int, Is>{}), ...);
}
// f(integral_constant<int, 0>) ... f(integral_constant<int, N-1>), fully unrolled
template <int N, typename F> __device__ __forceinline__ void static_for(F &&f) {
  static_for_impl(std::make_integer_sequence<int, N>{}, static_cast<F &&>(f));
}

// LDS reads whose issue point is fixed by the program text (not by the scheduler).  The data is
// valid only after an lds_wait<N>() on the same registers, N = number of such reads issued after
// the one waited for (LDS reads complete in issue order).
template <int OFF> __device__ __forceinline__ u32x4 lds_b128(uint32_t addr) {
  u32x4 d;
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(d) : "v"(addr), "n"(OFF));
  return d;
}
template <int OFF> __device__ __forceinline__ u32x2 lds_tr64(uint32_t addr) {
  u32x2 d;
  asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(d) : "v"(addr), "n"(OFF));
  return d;
}
// x * alpha for a value that lives in a matrix-core accumulation register, done where it stands:
// the value never changes register class, so code paths that do not rescale carry no copies.
__device__ __forceinline__ float acc_scale(float x, float alpha) {
  float t;
  asm volatile("v_accvgpr_read_b32 %1, %0\n\tv_mul_f32 %1, %1, %2\n\ts_nop 1\n\tv_accvgpr_write_b32 %0, %1\n\ts_nop 1"
               : "+a"(x), "=&v"(t)
               : "v"(alpha));
  return x;
}
// pair_sum / pair_max (common.hpp) for use inside a rarely taken block of a hot loop.  The compiler treats
// the cross-lane builtin as a convergent operation, restructures the branch around it and then copies every
// accumulator on the path that skips the block; written as asm the exchange is an ordinary statement.
__device__ __forceinline__ void rare_pair(float x, float &lo, float &hi) {
  lo = x;
  hi = x;
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(lo), "+v"(hi));
}
__device__ __forceinline__ float rare_pair_sum(float x) {
  float lo, hi;
  rare_pair(x, lo, hi);
  return lo + hi;
}
__device__ __forceinline__ float rare_pair_max(float x) {
  float lo, hi;
  rare_pair(x, lo, hi);
  return fmaxf(lo, hi);
}

// (t, o) <- (alpha * (t + neg_shift * o), alpha * o) for two values that live in accumulation registers, done
// where they stand: the tangent accumulator is re-centred on a new reference for S' (see fwd_kernel_v2.hpp) and
// both follow a new reference point of the exponentials.
// The registers are named as inputs and written all the same.  That is sound only where nothing but in-place
// statements (mfma_acc, this one) touches the tiles from their first product to the end of the tile loop, so
// that the compiler never holds a value of theirs anywhere else.  (With the elements as in/out operands the
// compiler gives the tiles a second home after the rarely taken block this is used in, and copies all of
// them there on the path that skips the block, on every half tile.)
__device__ __forceinline__ void acc_move_in_place(float t, float o, float alpha, float neg_shift) {
  float a, b;
  asm volatile(
      "v_accvgpr_read_b32 %0, %2\n\tv_accvgpr_read_b32 %1, %3\n\tv_fma_f32 %0, %1, %5, %0\n\t"
      "v_mul_f32 %1, %1, %4\n\tv_mul_f32 %0, %0, %4\n\ts_nop 1\n\t"
      "v_accvgpr_write_b32 %3, %1\n\tv_accvgpr_write_b32 %2, %0\n\ts_nop 1"
      : "=&v"(a), "=&v"(b)
      : "a"(t), "a"(o), "v"(alpha), "v"(neg_shift)
      : "memory");
}
// Products whose B operand stays resident in the accumulation register file for the whole kernel
// while the result tile lives in ordinary vector registers: c = a*b (FIRST) or c += a*b.  The
// result may only be read by other instruction kinds after tiles_ready().
__device__ __forceinline__ void pin_acc(bf16x8 &f) { asm volatile("" : "+a"(f)); }
__device__ __forceinline__ void pin_acc(f16x8 &f) { asm volatile("" : "+a"(f)); }
// GUARD: two idle issue slots in front, for kernels whose resident operands fill the accumulation file
// to the last register, where the allocator moves them through a spare register right before their
// use (a matrix instruction must not read a register that soon after a vector-ALU write to it, and
// the compiler does not look inside inline asm).
template <bool FIRST, bool GUARD = false> __device__ __forceinline__ void mma_vra(f32x16 &c, const bf16x8 &a, const bf16x8 &b) {
  if constexpr (GUARD) {
    if constexpr (FIRST) asm("s_nop 1\n\tv_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(c) : "v"(a), "a"(b));
    else asm("s_nop 1\n\tv_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "a"(b));
  } else {
    if constexpr (FIRST) asm("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(c) : "v"(a), "a"(b));
    else asm("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "a"(b));
  }
}
template <bool FIRST, bool GUARD = false> __device__ __forceinline__ void mma_vra(f32x16 &c, const f16x8 &a, const f16x8 &b) {
  if constexpr (GUARD) {
    if constexpr (FIRST) asm("s_nop 1\n\tv_mfma_f32_32x32x16_f16 %0, %1, %2, 0" : "=&v"(c) : "v"(a), "a"(b));
    else asm("s_nop 1\n\tv_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "a"(b));
  } else {
    if constexpr (FIRST) asm("v_mfma_f32_32x32x16_f16 %0, %1, %2, 0" : "=&v"(c) : "v"(a), "a"(b));
    else asm("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "a"(b));
  }
}
// The same with the B operand in ordinary vector registers.  Under register pressure the compiler may
// park such a long-lived operand in the accumulation file and copy it back just before its use; a
// matrix instruction must not read a register within two issue slots of a vector-ALU write to it, and
// the compiler does not look inside inline asm, so the two slots are written here.
template <bool FIRST> __device__ __forceinline__ void mma_vrv(f32x16 &c, const bf16x8 &a, const bf16x8 &b) {
  if constexpr (FIRST) asm("s_nop 1\n\tv_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(c) : "v"(a), "v"(b));
  else asm("s_nop 1\n\tv_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "v"(b));
}
template <bool FIRST> __device__ __forceinline__ void mma_vrv(f32x16 &c, const f16x8 &a, const f16x8 &b) {
  if constexpr (FIRST) asm("s_nop 1\n\tv_mfma_f32_32x32x16_f16 %0, %1, %2, 0" : "=&v"(c) : "v"(a), "v"(b));
  else asm("s_nop 1\n\tv_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "v"(b));
}
// Accumulation in place: the tile is read and written in the same accumulation registers, so the
// register allocator can never give it a second home (and copy it there on the common path).
__device__ __forceinline__ void mfma_acc(f32x16 &c, const bf16x8 &a, const bf16x8 &b) {
  asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
}
__device__ __forceinline__ void mfma_acc(f32x16 &c, const f16x8 &a, const f16x8 &b) {
  asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
}
__device__ __forceinline__ void pin_acc(f32x16 &c) { asm volatile("" : "+a"(c)); }

// 32 idle issue slots behind the last in-place accumulation, tied to the tiles: code the compiler generates to
// read them (the epilogue) cannot be scheduled in front of the wait, which a bare asm statement would allow.
template <int N> __device__ __forceinline__ void accs_ready(f32x16 (&o)[N]) {
  static_assert(N == 1 || N == 2 || N == 4 || N == 8);
  if constexpr (N == 1) asm volatile("s_nop 15\n\ts_nop 15" : "+a"(o[0]));
  if constexpr (N == 2) asm volatile("s_nop 15\n\ts_nop 15" : "+a"(o[0]), "+a"(o[1]));
  if constexpr (N == 4) asm volatile("s_nop 15\n\ts_nop 15" : "+a"(o[0]), "+a"(o[1]), "+a"(o[2]), "+a"(o[3]));
  if constexpr (N == 8)
    asm volatile("s_nop 15\n\ts_nop 15"
                 : "+a"(o[0]), "+a"(o[1]), "+a"(o[2]), "+a"(o[3]), "+a"(o[4]), "+a"(o[5]), "+a"(o[6]), "+a"(o[7]));
}
template <int N> __device__ __forceinline__ void accs_ready(f32x16 (&o)[N], f32x16 (&t)[N]) {
  static_assert(N == 1 || N == 2 || N == 4);
  if constexpr (N == 1) asm volatile("s_nop 15\n\ts_nop 15" : "+a"(o[0]), "+a"(t[0]));
  if constexpr (N == 2) asm volatile("s_nop 15\n\ts_nop 15" : "+a"(o[0]), "+a"(o[1]), "+a"(t[0]), "+a"(t[1]));
  if constexpr (N == 4)
    asm volatile("s_nop 15\n\ts_nop 15"
                 : "+a"(o[0]), "+a"(o[1]), "+a"(o[2]), "+a"(o[3]), "+a"(t[0]), "+a"(t[1]), "+a"(t[2]), "+a"(t[3]));
}

// 16 + 4 idle issue slots: the last matrix-core pass has written its registers when this returns
__device__ __forceinline__ void tiles_ready(f32x16 &a) { asm volatile("s_nop 15\n\ts_nop 3" : "+v"(a)); }
__device__ __forceinline__ void tiles_ready(f32x16 &a, f32x16 &b) {
  asm volatile("s_nop 15\n\ts_nop 3" : "+v"(a), "+v"(b));
}
__device__ __forceinline__ void tiles_ready(f32x16 &a, f32x16 &b, f32x16 &c, f32x16 &d) {
  asm volatile("s_nop 15\n\ts_nop 3" : "+v"(a), "+v"(b), "+v"(c), "+v"(d));
}
template <int N> __device__ __forceinline__ void lds_wait(u32x4 &a) {
  asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(a) : "n"(N));
}
template <int N> __device__ __forceinline__ void lds_wait(u32x4 &a, u32x4 &b) {
  asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(a), "+v"(b) : "n"(N));
}
template <int N> __device__ __forceinline__ void lds_wait(u32x2 &a, u32x2 &b) {
  asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(a), "+v"(b) : "n"(N));
}
template <int N> __device__ __forceinline__ void lds_wait(u32x2 &a, u32x2 &b, u32x2 &c, u32x2 &d) {
  asm volatile("s_waitcnt lgkmcnt(%4)" : "+v"(a), "+v"(b), "+v"(c), "+v"(d) : "n"(N));
}

// One int of a list in global memory, read a whole tile before it is needed.  list_request is a
// plain load, issued where it is written (memory operations are not moved across the inline-asm
// matrix instructions and LDS reads around it); list_take, placed where the value is first needed,
// moves it to a scalar register.  Being inline asm it stays put as well, so the wait for the load
// (which the compiler inserts in front of it) lands there and not in the middle of the tile, where
// it would also wait for every older load still in flight.  p must be the same address in every
// lane.
__device__ __forceinline__ int list_request(const int *p) { return *p; }
__device__ __forceinline__ int list_take(int v) {
  int s;
  asm volatile("v_readfirstlane_b32 %0, %1\n\ts_nop 4" : "=s"(s) : "v"(v));
  return s;
}

// chunk swizzles (row -> xor value applied to the 16-byte chunk index)
//
// The LDS has 64 banks of 4 bytes.  A ds_read_b128 is served 16 lanes at a time (16 x 16 bytes = all banks
// once if the 16 lanes, which read 16 consecutive rows at one logical chunk, land in 16 different chunks of
// a 256-byte line); a ds_read_b64_tr_b16 is served 32 lanes at a time: the lanes 16a + j of a half wave
// read row 4hh + j/4, the 8-byte half (j/2)%2 of logical chunk 4db + 2a + j%2, so the four rows j/4 must
// move the chunk index in bits that neither a nor j%2 occupies (bits 2 and up), or two lanes of the half
// wave meet in a bank and the read takes twice as long (measured before: 2 conflict cycles per
// transposing read, 33 % of the LDS cycles of the headline forward).
// (CH = 4, rows of 64 bytes: four rows share a line of 256 bytes, which the transposing read of four
// consecutive rows covers exactly, so only the row-wise read needs its chunks moved)
template <int CH> __device__ __forceinline__ int swz_k(int row) {
  return (CH == 32 || CH == 16) ? (row & 15) : CH == 8 ? ((row >> 1) & 7) : ((row >> 2) & 3);
}
// Tiles read by the transposing read only.  (CH = 32, 16: every row starts a 256-byte line, rows 0..3 move
// bits 2-3; CH = 8: two rows share a line and differ in the bank already, rows 2-3 move bit 2.)
template <int CH> __device__ __forceinline__ int swz_v(int row) {
  return (CH == 32 || CH == 16) ? ((row & 3) << 2) : CH == 8 ? (((row >> 1) & 1) << 2) : 0;
}

// Swizzle for tiles that are read both ways: 16 consecutive rows (8 pairs for CH = 8) get different values
// for the row-wise read, and the rows j/4 of a transposing read move bits 2 and up.
template <int CH> __device__ __forceinline__ int swz_u(int row) {
  if (CH == 16) return ((row & 3) << 2) | ((row >> 2) & 3);
  if (CH == 4) return (row >> 2) & 3;
  const int x = (row >> 1) & 7;
  return ((x & 1) << 2) | (x >> 1);
}

}  // namespace jvpfa
