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
//                6  vector ALU  register-only loops of one instruction (DECA_OP), 16 independent
//                               chains per lane, and of an MFMA with vector work behind it
//   DECA_THREADS    lanes per workgroup
//   DECA_CHUNKS     (0..2) 16-byte chunks of the buffer; DECA_UNROLL accesses in flight per lane;
//                   DECA_NT 1: non-temporal loads / stores
//   DECA_ITERS      (3, 4) loop trips, DECA_NACC independent accumulator tiles per wave
#include <hip/hip_runtime.h>

#pragma clang diagnostic ignored "-Winline-asm"  // M0 is set and declared clobbered on purpose

typedef float f4 __attribute__((ext_vector_type(4)));
typedef float f16v __attribute__((ext_vector_type(16)));
typedef _Float16 half8 __attribute__((ext_vector_type(8)));

#if DECA_CEILING == 6
// DECA_OP 0 v_fma_f32, 1 v_exp_f32, 2 v_cvt_pk_f16_f32 (packs two results), 3 v_max3_f32,
// 4 one 32x32x16 MFMA (zero operands) followed by two v_exp_f32 in the same wave, 5 the same
// with eight v_fma_f32, 6 the MFMAs alone, 7 an MFMA followed by the softmax mix of a
// FlashAttention tile (2 fma, 1 exp, 1 cvt_pk, 1 max3), 8 that mix twice per MFMA (head
// dim 64), 9 the same plus two reads of accumulation registers,
// 10-12 sixteen v_fma_f32 / v_exp_f32 / v_max3_f32 that each consume the one before, 13 sixteen
// v_exp_f32 each followed by a v_add_f32 that consumes it; DECA_ACC_AGPR 1 keeps the MFMA accumulators in
// the accumulation half of the register file
extern "C" __global__ void __launch_bounds__(256)
deca_main(const float* __restrict__ in, float* __restrict__ out) {
  float x[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) x[i] = in[(threadIdx.x + i * 256) % 4096];
  const float c0 = in[threadIdx.x], c1 = in[threadIdx.x + 1];
#if DECA_OP >= 4
  half8 a, b;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    a[i] = static_cast<_Float16>(in[4096 + (threadIdx.x + i) % 4096]);  // the host keeps this half zero:
    b[i] = static_cast<_Float16>(in[4096 + (threadIdx.x * 3 + i) % 4096]);  // no power limit on the MFMAs
  }
  f16v acc[4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[i][e] = 0.f;
#endif
  for (int it = 0; it < DECA_ITERS; ++it) {
#if DECA_OP >= 10
    // one dependent chain: what a wave waits between an instruction and its consumer
#pragma unroll
    for (int i = 0; i < 16; ++i) {
#if DECA_OP == 10
      asm volatile("v_fma_f32 %0, %0, %1, %2" : "+v"(x[0]) : "v"(c0), "v"(c1));
#elif DECA_OP == 11
      asm volatile("v_exp_f32 %0, %0" : "+v"(x[0]));
#elif DECA_OP == 12
      asm volatile("v_max3_f32 %0, %0, %1, %2" : "+v"(x[0]) : "v"(c0), "v"(c1));
#else
      asm volatile("v_exp_f32 %0, %0\n\tv_add_f32 %1, %1, %0" : "+v"(x[i]), "+v"(x[(i + 1) % 16]));
#endif
    }
#elif DECA_OP < 4
#pragma unroll
    for (int i = 0; i < 16; ++i) {
#if DECA_OP == 0
      asm volatile("v_fma_f32 %0, %0, %1, %2" : "+v"(x[i]) : "v"(c0), "v"(c1));
#elif DECA_OP == 1
      asm volatile("v_exp_f32 %0, %0" : "+v"(x[i]));
#elif DECA_OP == 2
      asm volatile("v_cvt_pk_f16_f32 %0, %0, %1" : "+v"(x[i]) : "v"(c0));
#else
      asm volatile("v_max3_f32 %0, %0, %1, %2" : "+v"(x[i]) : "v"(c0), "v"(c1));
#endif
    }
#else
#pragma unroll
    for (int i = 0; i < 4; ++i) {
#if DECA_ACC_AGPR
      asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+a"(acc[i]) : "v"(a), "v"(b));
#else
      acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, acc[i], 0, 0, 0);
#endif
#if DECA_OP == 4
      asm volatile("v_exp_f32 %0, %0\n\tv_exp_f32 %1, %1" : "+v"(x[2 * i]), "+v"(x[2 * i + 1]));
#elif DECA_OP == 7
      asm volatile("v_fma_f32 %0, %0, %4, %5\n\tv_exp_f32 %1, %1\n\tv_fma_f32 %2, %2, %4, %5\n\t"
                   "v_cvt_pk_f16_f32 %3, %3, %4\n\tv_max3_f32 %0, %0, %4, %5"
                   : "+v"(x[4 * i]), "+v"(x[4 * i + 1]), "+v"(x[4 * i + 2]), "+v"(x[4 * i + 3])
                   : "v"(c0), "v"(c1));
#elif DECA_OP == 8 || DECA_OP == 9
#pragma unroll
      for (int j = 0; j < 2; ++j)
        asm volatile("v_fma_f32 %0, %0, %4, %5\n\tv_exp_f32 %1, %1\n\tv_fma_f32 %2, %2, %4, %5\n\t"
                     "v_cvt_pk_f16_f32 %3, %3, %4\n\tv_max3_f32 %0, %0, %4, %5"
                     : "+v"(x[4 * i]), "+v"(x[4 * i + 1]), "+v"(x[4 * i + 2]), "+v"(x[4 * i + 3])
                     : "v"(c0), "v"(c1));
#if DECA_OP == 9 && DECA_ACC_AGPR
      // (timing probe only: the accumulator read here was written two MFMAs earlier, with
      // no wait states placed by hand -- what it reads is not used as a value)
      asm volatile("v_accvgpr_read_b32 %0, %2\n\tv_accvgpr_read_b32 %1, %3"
                   : "=v"(x[(4 * i + 5) % 16]), "=v"(x[(4 * i + 6) % 16]) : "a"(acc[(i + 2) % 4][0]), "a"(acc[(i + 2) % 4][1]));
#endif
#elif DECA_OP == 5
#pragma unroll
      for (int j = 0; j < 8; ++j)
        asm volatile("v_fma_f32 %0, %0, %1, %2" : "+v"(x[(4 * i + j) % 16]) : "v"(c0), "v"(c1));
#endif
    }
#endif
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 16; ++i) s += x[i];
#if DECA_OP >= 4
#if DECA_ACC_AGPR
  // The MFMAs above are inline assembly: the compiler places no wait states between the
  // last of them and the reads of their results below (18 are owed after a 16-pass MFMA).
  __builtin_amdgcn_sched_barrier(0);
  asm volatile("s_nop 15\n\ts_nop 3" ::: "memory");
  __builtin_amdgcn_sched_barrier(0);
#endif
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int e = 0; e < 16; ++e) s += acc[i][e];
#endif
  out[blockIdx.x * 256 + threadIdx.x] = s;
}
#elif DECA_CEILING == 5
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
