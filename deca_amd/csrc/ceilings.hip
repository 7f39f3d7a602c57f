// Kernels that do nothing but the roofline-limited work, for measuring what the board
// sustains: the ceilings the cost model's constants and the roofline fractions are read
// against.  One code object per (DECA_CEILING, ...) specialisation, driven by
// deca_amd/arch/ceilings.py.
//
//   DECA_CEILING 0  copy        out[i] = in[i], 16 bytes per lane and access
//                1  read only   every lane sums what it reads; nothing is written
//                2  write only  16-byte stores of a lane-dependent constant
//                3  matrix      register-only loop of v_mfma_f32_32x32x16_f16
//                4  matrix      register-only loop of v_mfma_f32_16x16x32_f16
//   DECA_THREADS    lanes per workgroup
//   DECA_CHUNKS     (0..2) 16-byte chunks of the buffer; DECA_UNROLL accesses in flight per lane;
//                   DECA_NT 1: non-temporal loads / stores
//   DECA_ITERS      (3, 4) loop trips, DECA_NACC independent accumulator tiles per wave
#include <hip/hip_runtime.h>

typedef float f4 __attribute__((ext_vector_type(4)));
typedef float f16v __attribute__((ext_vector_type(16)));
typedef _Float16 half8 __attribute__((ext_vector_type(8)));

#if DECA_CEILING <= 2
extern "C" __global__ void __launch_bounds__(DECA_THREADS)
deca_main(const f4* __restrict__ in, f4* __restrict__ out) {
  const long tid = static_cast<long>(blockIdx.x) * DECA_THREADS + threadIdx.x;
  const long nthreads = static_cast<long>(gridDim.x) * DECA_THREADS;
  f4 acc = {0.f, 0.f, 0.f, 0.f};
  for (long base = tid; base < DECA_CHUNKS; base += nthreads * DECA_UNROLL) {
    f4 v[DECA_UNROLL];
#pragma unroll
    for (int u = 0; u < DECA_UNROLL; ++u) {
      const long i = base + u * nthreads;
      if (i >= DECA_CHUNKS) continue;
#if DECA_CEILING == 2
      v[u] = f4{1.f, 2.f, 3.f, static_cast<float>(i)};
#elif DECA_NT
      v[u] = __builtin_nontemporal_load(in + i);
#else
      v[u] = in[i];
#endif
    }
#pragma unroll
    for (int u = 0; u < DECA_UNROLL; ++u) {
      const long i = base + u * nthreads;
      if (i >= DECA_CHUNKS) continue;
#if DECA_CEILING == 1
      acc += v[u];
#elif DECA_NT
      __builtin_nontemporal_store(v[u], out + i);
#else
      out[i] = v[u];
#endif
    }
  }
#if DECA_CEILING == 1
  // never true for finite data; keeps the loads alive
  if (acc.x + acc.y + acc.z + acc.w == 12345.678f && tid < DECA_CHUNKS) out[tid] = acc;
#endif
}
#else
// `in` holds 4096 half8 operand values; each wave keeps DECA_NACC accumulator tiles busy
// with operands that never change, so that nothing but the matrix pipe limits the loop.
extern "C" __global__ void __launch_bounds__(DECA_THREADS)
deca_main(const half8* __restrict__ in, float* __restrict__ out) {
  half8 a[4], b[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    a[i] = in[(threadIdx.x + i * 256) % 4096];
    b[i] = in[(threadIdx.x * 7 + i * 131) % 4096];
  }
#if DECA_CEILING == 3
  f16v acc[DECA_NACC];
  constexpr int REGS = 16;
#else
  f4 acc[DECA_NACC];
  constexpr int REGS = 4;
#endif
#pragma unroll
  for (int i = 0; i < DECA_NACC; ++i)
#pragma unroll
    for (int e = 0; e < REGS; ++e) acc[i][e] = 0.f;
  for (int it = 0; it < DECA_ITERS; ++it) {
#pragma unroll
    for (int i = 0; i < DECA_NACC; ++i) {
#if DECA_CEILING == 3
      acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[i % 4], b[(i / 4) % 4], acc[i], 0, 0, 0);
#else
      acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[i % 4], b[(i / 4) % 4], acc[i], 0, 0, 0);
#endif
    }
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < DECA_NACC; ++i)
#pragma unroll
    for (int e = 0; e < REGS; ++e) s += acc[i][e];
  out[blockIdx.x * DECA_THREADS + threadIdx.x] = s;
}
#endif
