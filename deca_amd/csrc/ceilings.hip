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
//                5  LDS / L2    8 waves per workgroup: DECA_READERS of them stream conflict-free
//                               ds_read_b128, DECA_LOADERS stream direct global->LDS loads
//                               (global_load_lds_dwordx4) from a 4 MiB, L2-resident region,
//                               DECA_ITERS trips of 8 KiB per wave each
//   DECA_THREADS    lanes per workgroup
//   DECA_CHUNKS     (0..2) 16-byte chunks of the buffer; DECA_UNROLL accesses in flight per lane;
//                   DECA_NT 1: non-temporal loads / stores
//   DECA_ITERS      (3, 4) loop trips, DECA_NACC independent accumulator tiles per wave
#include <hip/hip_runtime.h>

#pragma clang diagnostic ignored "-Winline-asm"  // M0 is set and declared clobbered on purpose

typedef float f4 __attribute__((ext_vector_type(4)));
typedef float f16v __attribute__((ext_vector_type(16)));
typedef _Float16 half8 __attribute__((ext_vector_type(8)));

#if DECA_CEILING == 5
extern "C" __global__ void __launch_bounds__(512)
deca_main(const unsigned char* __restrict__ in, float* __restrict__ out) {
  __shared__ __attribute__((aligned(16))) unsigned char lds[128 * 1024];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  for (int i = threadIdx.x; i < 32768; i += 512) reinterpret_cast<float*>(lds)[i] = static_cast<float>(i);
  __syncthreads();
  f4 acc = {0.f, 0.f, 0.f, 0.f};
  if (wave < DECA_READERS) {
    const unsigned char* p = lds + wave * 8192 + lane * 16;
    for (int it = 0; it < DECA_ITERS; ++it) {
#pragma unroll
      for (int u = 0; u < 8; ++u) acc += *reinterpret_cast<const f4*>(p + u * 1024);
    }
  } else if (wave < DECA_READERS + DECA_LOADERS) {
    // lane L's 16 bytes land at (wave-uniform LDS base in M0) + 16 L
    const unsigned dst = static_cast<unsigned>(reinterpret_cast<size_t>(
        (__attribute__((address_space(3))) void*)(lds + 65536 + (wave - DECA_READERS) * 8192)));
    const unsigned voff = lane * 16;
    const unsigned char* src = in + (blockIdx.x & 63) * 65536 + (wave - DECA_READERS) * 8192;
    for (int it = 0; it < DECA_ITERS; ++it) {
#pragma unroll
      for (int u = 0; u < 8; ++u)
        asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                     :
                     : "v"(voff), "s"(src + u * 1024), "s"(dst + u * 1024)
                     : "memory", "m0");
      __builtin_amdgcn_s_waitcnt(0x0F78);  // vmcnt(8): one trip stays in flight
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
  }
  __syncthreads();
  out[blockIdx.x * 512 + threadIdx.x] = acc.x + acc.y + acc.z + acc.w + lds[threadIdx.x * 4 + 65536];
}
#elif DECA_CEILING <= 2
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
