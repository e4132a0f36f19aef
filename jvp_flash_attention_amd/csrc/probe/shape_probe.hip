// Issue model of three shapes of the dual forward at D = 128 (no data meaning: instruction mix only).
//   A: four 32-row waves per workgroup, one per SIMD, v_mfma_f32_32x32x16_bf16; per matrix instruction one
//      1 KB LDS fragment read (four ahead), three fma-class vector instructions, a quarter exponential.
//   B: eight 16-row waves, two per SIMD, v_mfma_f32_16x16x32_bf16 (half the flops each); per matrix
//      instruction one fragment read, 1.5 vector instructions, an eighth of an exponential.
//   C: four 64-row waves, one per SIMD, 32x32x16; a fragment read serves two matrix instructions.
// Time is reported per 128 query rows x 32 keys of work on one compute unit (48 32x32x16 matrix
// instructions per SIMD = 1536 cycles of matrix pipe).
#include <hip/hip_runtime.h>
#include <cstdio>
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) unsigned u32x4;

template <int SHAPE, int VALU_PCT>  // VALU_PCT: 100 = the mix above, 0 = no vector instructions
__global__ __launch_bounds__(SHAPE == 1 ? 512 : 256) void k(float* out, int iters) {
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
  const unsigned lds0 = (unsigned)(uintptr_t)smem;
  const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
  bf16x8 a;
  for (int i = 0; i < 8; ++i) a[i] = (__bf16)(float)(threadIdx.x + i);
  f32x16 c0, c1, c2, c3;
  f32x4 d0, d1, d2, d3;
  for (int i = 0; i < 16; ++i) { c0[i] = 0; c1[i] = 0; c2[i] = 0; c3[i] = 0; }
  for (int i = 0; i < 4; ++i) { d0[i] = 0; d1[i] = 0; d2[i] = 0; d3[i] = 0; }
  asm volatile("" : "+a"(c0), "+a"(c1), "+a"(c2), "+a"(c3));
  asm volatile("" : "+a"(d0), "+a"(d1), "+a"(d2), "+a"(d3));
  // every wave reads the same 32 KB tile region (as the waves of a workgroup do), conflict-free rows
  const unsigned ad = lds0 + (lane % 16) * 256 + ((lane / 16) ^ (lane % 16)) * 16;
  constexpr int AHEAD = 4, RING = AHEAD + 1;
  u32x4 r[RING];
  for (int i = 0; i < RING; ++i) r[i] = u32x4{0, 0, 0, 0};
  float v[8];
  for (int i = 0; i < 8; ++i) v[i] = 1.f + 1e-3f * (lane + i);
  const float m1 = 0.999f, m2 = 1e-4f;
  // vector instructions per group in eighths: A 24 fma + 2 exp, B 12 + 1, C 48 + 4
  constexpr int FMA8 = (SHAPE == 0 ? 24 : SHAPE == 1 ? 12 : 48) * VALU_PCT / 100;
  constexpr int EXP8 = (SHAPE == 0 ? 2 : SHAPE == 1 ? 1 : 4) * VALU_PCT / 100;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int u = 0; u < RING * 8; ++u) {  // 40 groups per trip
      const int sl = u % RING, nx = (u + AHEAD) % RING;
      asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(r[sl]) : "n"(AHEAD - 1));
      asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(r[nx]) : "v"(ad), "n"((u % 8) * 4096));
      const bf16x8 b = __builtin_bit_cast(bf16x8, r[sl]);
      if constexpr (SHAPE == 1) {
        if (u & 1) asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(d0) : "v"(a), "v"(b));
        else asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(d1) : "v"(a), "v"(b));
      } else {
        if (u & 1) asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(c0) : "v"(a), "v"(b));
        else asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(c1) : "v"(a), "v"(b));
      }
      // this group's share of the vector work (the count over 8 groups is exact)
      const int f_lo = (u % 8) * FMA8 / 8, f_hi = (u % 8 + 1) * FMA8 / 8;
      const int e_lo = (u % 8) * EXP8 / 8, e_hi = (u % 8 + 1) * EXP8 / 8;
      const int nf = f_hi - f_lo, ne = e_hi - e_lo;
      // C: half of the vector work in front of the second matrix instruction, half behind it
      const int nf_first = SHAPE == 2 ? nf / 2 : nf;
#pragma unroll
      for (int j = 0; j < nf_first; ++j) asm volatile("v_fma_f32 %0, %0, %1, %2" : "+v"(v[(f_lo + j) % 8]) : "v"(m1), "v"(m2));
      if constexpr (SHAPE == 2) {
        if (u & 1) asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(c2) : "v"(a), "v"(b));
        else asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(c3) : "v"(a), "v"(b));
#pragma unroll
        for (int j = nf_first; j < nf; ++j) asm volatile("v_fma_f32 %0, %0, %1, %2" : "+v"(v[(f_lo + j) % 8]) : "v"(m1), "v"(m2));
      }
#pragma unroll
      for (int j = 0; j < ne; ++j) asm volatile("v_exp_f32 %0, %0" : "+v"(v[(e_lo + j + 4) % 8]));
    }
  }
  float s = 0;
  for (int i = 0; i < 8; ++i) s += v[i];
  for (int i = 0; i < 16; ++i) s += c0[i] + c1[i] + c2[i] + c3[i];
  for (int i = 0; i < 4; ++i) s += d0[i] + d1[i] + d2[i] + d3[i];
  out[blockIdx.x * 512 + threadIdx.x] = s;
}
template <int SHAPE, int VALU_PCT> void run(float* d, const char* name) {
  hipEvent_t e0, e1; (void)hipEventCreate(&e0); (void)hipEventCreate(&e1);
  const int iters = 40000, threads = SHAPE == 1 ? 512 : 256;
  auto kern = k<SHAPE, VALU_PCT>;
  (void)hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, 65536);
  kern<<<256, threads, 65536>>>(d, 10);
  float ms = 1e30f;
  for (int rep = 0; rep < 5; ++rep) {  // the fastest of five launches (the clock settles during the first)
    (void)hipEventRecord(e0);
    kern<<<256, threads, 65536>>>(d, iters);
    (void)hipEventRecord(e1); (void)hipEventSynchronize(e1);
    float t; (void)hipEventElapsedTime(&t, e0, e1);
    ms = t < ms ? t : ms;
  }
  // groups per wave: iters * 40.  Work unit = 128 rows x 32 keys per compute unit:
  // A: 48 groups of each of 4 waves; B: 48 groups of each of 8 waves (96 per SIMD); C: 48 groups (96 MFMAs) cover 256 rows -> 24 groups
  const double groups = iters * 40.0, per_unit = SHAPE == 2 ? 24.0 : 48.0;
  const double ns_unit = ms * 1e6 / groups * per_unit;
  printf("%-34s vector work %3d %%: %7.1f ns per 128 rows x 32 keys\n", name, VALU_PCT, ns_unit); fflush(stdout);
}
int main() {
  float* d; (void)hipMalloc(&d, 256 * 512 * 4);
  run<0, 0>(d, "A 4 x 32-row waves, 32x32x16");
  run<0, 100>(d, "A 4 x 32-row waves, 32x32x16");
  run<0, 150>(d, "A 4 x 32-row waves, 32x32x16");
  run<1, 0>(d, "B 8 x 16-row waves, 16x16x32");
  run<1, 100>(d, "B 8 x 16-row waves, 16x16x32");
  run<1, 150>(d, "B 8 x 16-row waves, 16x16x32");
  run<2, 0>(d, "C 4 x 64-row waves, 32x32x16");
  run<2, 100>(d, "C 4 x 64-row waves, 32x32x16");
  run<2, 150>(d, "C 4 x 64-row waves, 32x32x16");
  return 0;
}
