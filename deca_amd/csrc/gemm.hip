// 16-bit x 16-bit -> fp32-accumulate GEMM, C[M,N] = A[M,K] * B[K,N], all row-major
// float16 (or bfloat16 with DECA_BF16), for gfx950 (MFMA v_mfma_f32_32x32x16_f16 /
// _bf16).
//
// One code object per (shape, GemmConfig); every DECA_* macro is a compile-time
// constant supplied by kernels/gemm_hip.py, as the reference bakes shape and
// config into each generated kernel (src/kernels/gemm_tir.py:123-156).
//
//   DECA_M/N/K    problem size          DECA_BM/BN/BK  workgroup tile
//   DECA_WM/WN    wave tile             DECA_STAGES    LDS ring depth (1 or 2)
//   DECA_RASTER   workgroup rows per rasterisation group; 0: 16 x 16 blocks of tiles,
//                 an 8 x 4 sub-block per XCD
//   DECA_EPI_LDS  1: stage C through LDS for 16-byte stores
//   DECA_XCD      1: remap workgroup ids so that each of the 8 XCDs (private L2)
//                 owns a contiguous slab of tiles
//   DECA_DIRECT   1: global -> LDS loads that bypass the VGPRs, ring of
//                 DECA_STAGES (2..4) tiles; 0: loads staged through VGPRs one
//                 tile ahead, ring of 1 or 2 tiles
//
// Data path (what the reference does with cp.async + ldmatrix + mma.sync,
// gemm_tir.py:190-334):
//   global -> LDS, either directly (global_load_lds_dwordx4, asynchronous,
//   counted by vmcnt like cp.async groups) or through VGPRs (16-byte loads
//   issued one K-tile ahead, then ds_write_b128), XOR-swizzled chunks
//   -> fragments, double buffered in registers one k-step ahead: A by ds_read_b128
//   (8 consecutive k per lane), B by ds_read_b64_tr_b16 (transposing read, so
//   the row-major [k][n] tile feeds the k-packed MFMA operand directly)
//   -> MFMA 32x32x16 with the operand roles swapped (B fragment as the first
//   operand) so that each lane ends up with 4 consecutive n of one row of C.
#include <hip/hip_runtime.h>

#ifndef DECA_BM
#error "gemm.hip is a template: define the DECA_* macros"
#endif
#ifndef DECA_MIN_WAVES
#define DECA_MIN_WAVES 1  // waves per SIMD the register allocation must leave room for
#endif
#ifndef DECA_BF16
#define DECA_BF16 0
#endif

#define M_ DECA_M
#define N_ DECA_N
#define K_ DECA_K
#define BM DECA_BM
#define BN DECA_BN
#define BK DECA_BK
#define WM DECA_WM
#define WN DECA_WN
#define STAGES DECA_STAGES

constexpr int WAVES_M = BM / WM;
constexpr int WAVES_N = BN / WN;
constexpr int NT = WAVES_M * WAVES_N * 64;
constexpr int MT = WM / 32;  // 32x32 MFMA tiles per wave along m
constexpr int NTL = WN / 32; // ... along n
constexpr int KS = BK / 16;  // MFMA k-steps per K-tile
constexpr int NK = K_ / BK;
constexpr int GM = M_ / BM;
constexpr int GN = N_ / BN;
constexpr int CPR_A = BK / 8;  // 16-byte chunks per A row in LDS
constexpr int CPR_B = BN / 8;  // ... per B row
constexpr int A_CHUNKS = BM * CPR_A;
constexpr int B_CHUNKS = BK * CPR_B;
constexpr int A_IT = A_CHUNKS / NT;
constexpr int B_IT = B_CHUNKS / NT;
constexpr int A_STAGE_BYTES = A_CHUNKS * 16;
constexpr int B_STAGE_BYTES = B_CHUNKS * 16;
constexpr int PIPE_BYTES = STAGES * (A_STAGE_BYTES + B_STAGE_BYTES);
constexpr int EPI_PAD = 8;  // halves; keeps the rows of the staged C tile on different banks
constexpr int EPI_BYTES = DECA_EPI_LDS ? BM * (BN + EPI_PAD) * 2 : 0;
constexpr int LDS_BYTES = PIPE_BYTES > EPI_BYTES ? PIPE_BYTES : EPI_BYTES;

static_assert(M_ % BM == 0 && N_ % BN == 0 && K_ % BK == 0, "tiles must divide the problem");
static_assert(BM % WM == 0 && BN % WN == 0 && WM % 32 == 0 && WN % 32 == 0, "wave tiles");
static_assert(BK % 16 == 0 && (CPR_A == 4 || CPR_A == 8), "BK must be 32 or 64");
static_assert(A_CHUNKS % NT == 0 && B_CHUNKS % NT == 0, "loader coverage");
static_assert(NT >= 64 && NT <= 1024, "workgroup size");
static_assert(STAGES >= 1 && STAGES <= 4, "LDS ring depth");
static_assert(DECA_DIRECT == 0 || STAGES >= 2, "the direct-to-LDS ring needs two slots");
static_assert(DECA_RASTER == 0 || GM % (DECA_RASTER ? DECA_RASTER : 1) == 0,
              "raster group must divide the workgroup rows");
static_assert(LDS_BYTES <= 160 * 1024, "LDS budget");
static_assert(CPR_B >= 8, "BN >= 64");

#if DECA_BF16
typedef __bf16 elem_t;
#define DECA_MFMA __builtin_amdgcn_mfma_f32_32x32x16_bf16
#else
typedef _Float16 elem_t;
#define DECA_MFMA __builtin_amdgcn_mfma_f32_32x32x16_f16
#endif
typedef elem_t half8 __attribute__((ext_vector_type(8)));
typedef elem_t half4 __attribute__((ext_vector_type(4)));
typedef short short4v __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) short4v* lds_s4_ptr;
typedef const __attribute__((address_space(1))) void* gptr;
typedef __attribute__((address_space(3))) void* lptr;

// ---- LDS layouts -----------------------------------------------------------
// A tile: [BM][BK] halves, k contiguous; 16-byte chunk c of row r sits at chunk
// slot c ^ f(r), f chosen so that 16 consecutive rows at one logical chunk
// cover all sixteen 16-byte bank groups of the 256-byte bank window.
__device__ __forceinline__ int a_chunk_slot(int row, int c) {
  constexpr int ROWS_PER_WINDOW = 16 / CPR_A;
  return row * CPR_A + (c ^ ((row / ROWS_PER_WINDOW) % CPR_A));
}
// B tile: [BK][BN] halves, n contiguous; 64-byte groups of a row are rotated by
// k % 4 so that the 4 k-rows of one transposing read hit different banks.
__device__ __forceinline__ int b_chunk_slot(int k, int c) {
  constexpr int MASK = CPR_B - 1;
  return k * CPR_B + (c ^ (((k & 3) << 2) & MASK));
}

extern "C" __global__ void __launch_bounds__(NT, DECA_MIN_WAVES)
deca_main(const elem_t* __restrict__ A, const elem_t* __restrict__ B,
          elem_t* __restrict__ C) {
  __shared__ __attribute__((aligned(16))) unsigned char lds[LDS_BYTES];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm0 = (wave / WAVES_N) * WM;
  const int wn0 = (wave % WAVES_N) * WN;

  // ---- workgroup -> tile mapping --------------------------------------------
  int lin = blockIdx.x;
#if DECA_RASTER == 0
  // Workgroups are dealt round-robin to the 8 XCDs.  The 256 workgroups in flight
  // (one per CU) form a 16 x 16 block of tiles, of which every XCD takes an 8 x 4
  // sub-block: its L2 fetches 12 operand panels for 32 tiles, and the 8 L2s
  // together ask the fabric for only 16 A and 16 B panels per 256 tiles.  Blocks
  // are walked row by row, back and forth, so that consecutive blocks share
  // their A panels, or at the turn their B panels.
  static_assert(GM % 16 == 0 && GN % 16 == 0, "16 x 16 blocks of tiles");
  static_assert(DECA_XCD, "the block order is an XCD order");
  int bm, bn;
  {
    const int x = lin & 7, idx = lin >> 3;
    const int sb = idx >> 5, within = idx & 31;
    constexpr int SBN = GN / 16;
    const int sbr = sb / SBN;
    int sbc = sb % SBN;
    if (sbr & 1) sbc = SBN - 1 - sbc;
    bm = sbr * 16 + (x >> 2) * 8 + (within & 7);
    bn = sbc * 16 + (x & 3) * 4 + (within >> 3);
  }
#else
#if DECA_XCD
  {
    // Workgroups are dealt round-robin to the 8 XCDs; give each XCD a
    // contiguous range of tiles so that its L2 sees a compact set of A rows
    // and B columns.
    constexpr int TILES = GM * GN;
    static_assert(TILES % 8 == 0, "XCD remap needs a multiple of 8 workgroups");
    lin = (lin & 7) * (TILES / 8) + (lin >> 3);
  }
#endif
  constexpr int GROUP = DECA_RASTER * GN;
  const int bm = (lin / GROUP) * DECA_RASTER + (lin % GROUP) % DECA_RASTER;
  const int bn = (lin % GROUP) / DECA_RASTER;
#endif

  const elem_t* a_gbase = A + static_cast<size_t>(bm) * BM * K_;
  const elem_t* b_gbase = B + static_cast<size_t>(bn) * BN;

  // ---- accumulators and fragment addressing -----------------------------------
  floatx16 acc[MT][NTL];
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int j = 0; j < NTL; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

  const int l32 = lane & 31;
  const int khalf = lane >> 5;
  // transposing B read: 16-lane block tb, lane ti in the block supplies the
  // address of row k0 + ti/4, columns n0 + 4*(ti%4) .. +3 and receives, for its
  // column n0 + ti, the four rows k0 .. k0+3
  const int tb = lane >> 4, ti = lane & 15;
  const int b_n_off = 16 * (tb & 1) + 4 * (ti & 3);  // + wn0 + nt * 32
  const int b_k_off = (tb >> 1) * 8 + (ti >> 2);     // + ks * 16 + r * 4

  // Fragments of k-step `ks` of the tile in ring slot `slot`.
  auto load_frags = [&](half8 (&af)[MT], half8 (&bf)[NTL], int slot, int ks) {
    const unsigned char* a_lds = lds + slot * A_STAGE_BYTES;
    const unsigned char* b_lds = lds + STAGES * A_STAGE_BYTES + slot * B_STAGE_BYTES;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const int row = wm0 + mt * 32 + l32;
      af[mt] = *reinterpret_cast<const half8*>(a_lds + a_chunk_slot(row, ks * 2 + khalf) * 16);
    }
#pragma unroll
    for (int nt = 0; nt < NTL; ++nt) {
      const int n = wn0 + nt * 32 + b_n_off;
      half4 h[2];
#pragma unroll
      for (int r = 0; r < 2; ++r) {
        const int k = ks * 16 + r * 4 + b_k_off;
        const unsigned char* p = b_lds + b_chunk_slot(k, n >> 3) * 16 + ((n >> 2) & 1) * 8;
        h[r] = __builtin_bit_cast(half4, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s4_ptr)(p)));
      }
      bf[nt] = __builtin_shufflevector(h[0], h[1], 0, 1, 2, 3, 4, 5, 6, 7);
    }
  };
  // Operand roles are swapped (B fragment first) so that a lane's four
  // consecutive accumulator registers are four consecutive n of one row of C.
  auto mfma_step = [&](const half8 (&af)[MT], const half8 (&bf)[NTL]) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int nt = 0; nt < NTL; ++nt)
        acc[mt][nt] = DECA_MFMA(bf[nt], af[mt], acc[mt][nt], 0, 0, 0);
  };

  // Scheduling pattern of one k-step: the LDS reads of the next fragments are
  // issued one per MFMA, so that they hide under the matrix pipe instead of
  // being grouped after it (mask 0x100 = DS read, 0x008 = MFMA).
  auto interleave_reads_with_mfma = [&]() {
    constexpr int READS = MT + 2 * NTL;
    constexpr int MFMAS = MT * NTL;
    constexpr int PAIRS = READS < MFMAS ? READS : MFMAS;
#pragma unroll
    for (int i = 0; i < PAIRS; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
    if (READS > PAIRS) __builtin_amdgcn_sched_group_barrier(0x100, READS - PAIRS, 0);
    if (MFMAS > PAIRS) __builtin_amdgcn_sched_group_barrier(0x008, MFMAS - PAIRS, 0);
  };

  half8 af0[MT], bf0[NTL], af1[MT], bf1[NTL];

#if DECA_DIRECT
  // ---- main loop: direct-to-LDS ring ---------------------------------------------
  // Tile kt lives in ring slot kt % STAGES.  Each lane issues LOADS 16-byte
  // global->LDS loads per tile; the hardware writes lane L's data to
  // (wave-uniform base) + L * 16, so the swizzle is applied by choosing which
  // global chunk each lane fetches.
  constexpr int LOADS = A_IT + B_IT;
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  const unsigned lds_u = static_cast<unsigned>(reinterpret_cast<size_t>((lptr)lds));
  // Byte offset of each lane's chunk from the tile's (wave-uniform) origin.
  unsigned a_voff[A_IT], b_voff[B_IT];
#pragma unroll
  for (int it = 0; it < A_IT; ++it) {
    const int sidx = it * NT + tid;
    const int row = sidx / CPR_A;
    const int c = (sidx % CPR_A) ^ ((row / (16 / CPR_A)) % CPR_A);
    a_voff[it] = static_cast<unsigned>(row * K_ + c * 8) * 2u;
  }
#pragma unroll
  for (int it = 0; it < B_IT; ++it) {
    const int sidx = it * NT + tid;
    const int k = sidx / CPR_B;
    const int c = (sidx % CPR_B) ^ (((k & 3) << 2) & (CPR_B - 1));
    b_voff[it] = static_cast<unsigned>(k * N_ + c * 8) * 2u;
  }
  static_assert(static_cast<long long>(BM) * K_ * 2 < (1ll << 32) &&
                static_cast<long long>(BK) * N_ * 2 < (1ll << 32), "32-bit lane offsets");
  // The load is written as inline assembly so that the compiler's wait-count
  // insertion does not see an LDS write and force vmcnt(0) before every LDS
  // read; the waits are explicit (DECA_WAIT_VMCNT) and paired with a barrier.
  // The "memory" clobber keeps LDS reads from moving across the issue point.
  auto dma16 = [&](const elem_t* origin, unsigned voff, unsigned lds_addr) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                 :
                 : "v"(voff), "s"(origin), "s"(lds_addr)
                 : "memory");
  };
  auto issue_tile = [&](int kt, int slot) {
    const elem_t* a_origin = a_gbase + kt * BK;
    const elem_t* b_origin = b_gbase + static_cast<size_t>(kt) * BK * N_;
    const unsigned a_dst = lds_u + slot * A_STAGE_BYTES + wave_u * 1024;
    const unsigned b_dst = lds_u + STAGES * A_STAGE_BYTES + slot * B_STAGE_BYTES + wave_u * 1024;
#pragma unroll
    for (int it = 0; it < A_IT; ++it) dma16(a_origin, a_voff[it], a_dst + it * NT * 16);
#pragma unroll
    for (int it = 0; it < B_IT; ++it) dma16(b_origin, b_voff[it], b_dst + it * NT * 16);
  };
  // s_waitcnt on the vector-memory counter only (gfx9 encoding: vmcnt in bits
  // 3:0 and 15:14, expcnt 6:4 and lgkmcnt 11:8 left at "no wait").
#define DECA_WAIT_VMCNT(n) __builtin_amdgcn_s_waitcnt(((n) & 15) | (((n) >> 4) << 14) | 0x0F70)
  constexpr int PENDING = (STAGES - 2) * LOADS;  // loads that may stay in flight
  static_assert(PENDING <= 63, "vmcnt holds 6 bits");
  static_assert(NK >= STAGES, "K too short for the ring");

#pragma unroll
  for (int s = 0; s < STAGES - 1; ++s) issue_tile(s, s);
  DECA_WAIT_VMCNT(PENDING);
  __builtin_amdgcn_s_barrier();
  load_frags(af0, bf0, 0, 0);

  int slot = 0;
  for (int kt = 0; kt < NK; ++kt) {
    const bool more = kt + STAGES - 1 < NK;
    int fill = slot + STAGES - 1;
    if (fill >= STAGES) fill -= STAGES;
    if (more) issue_tile(kt + STAGES - 1, fill);
    int next = slot + 1;
    if (next == STAGES) next = 0;
    // k-steps 0 .. KS-2: fragments of step ks+1 are fetched under the MFMAs of ks
#pragma unroll
    for (int ks = 0; ks < KS - 1; ++ks) {
      if (ks & 1) {
        load_frags(af0, bf0, slot, ks + 1);
        mfma_step(af1, bf1);
      } else {
        load_frags(af1, bf1, slot, ks + 1);
        mfma_step(af0, bf0);
      }
      interleave_reads_with_mfma();
    }
    // Tile kt+1 must have landed for every lane of the workgroup, and every
    // wave must be done reading slot `slot` before the next iteration refills it.
    if (more) {
      DECA_WAIT_VMCNT(PENDING);
    } else {
      DECA_WAIT_VMCNT(0);
    }
    // all of this wave's LDS reads of slot `slot` have returned
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0) only
    __builtin_amdgcn_s_barrier();
    if (kt + 1 < NK) {
      if ((KS - 1) & 1) load_frags(af0, bf0, next, 0);
      else load_frags(af1, bf1, next, 0);
    }
    if ((KS - 1) & 1) mfma_step(af1, bf1);
    else mfma_step(af0, bf0);
    if (kt + 1 < NK) interleave_reads_with_mfma();
    slot = next;
  }
  static_assert(KS % 2 == 0, "fragment double buffer assumes an even number of k-steps");
#else
  // ---- main loop: VGPR-staged ring -------------------------------------------------
  u32x4 a_stage[A_IT];
  u32x4 b_stage[B_IT];
  auto load_global = [&](int kt) {
#pragma unroll
    for (int it = 0; it < A_IT; ++it) {
      const int id = it * NT + tid;
      const int row = id / CPR_A, c = id % CPR_A;
      a_stage[it] = *reinterpret_cast<const u32x4*>(a_gbase + static_cast<size_t>(row) * K_ +
                                                    kt * BK + c * 8);
    }
#pragma unroll
    for (int it = 0; it < B_IT; ++it) {
      const int id = it * NT + tid;
      const int row = id / CPR_B, c = id % CPR_B;
      b_stage[it] = *reinterpret_cast<const u32x4*>(
          b_gbase + static_cast<size_t>(kt * BK + row) * N_ + c * 8);
    }
  };
  auto store_lds = [&](int slot) {
    unsigned char* a_lds = lds + slot * A_STAGE_BYTES;
    unsigned char* b_lds = lds + STAGES * A_STAGE_BYTES + slot * B_STAGE_BYTES;
#pragma unroll
    for (int it = 0; it < A_IT; ++it) {
      const int id = it * NT + tid;
      *reinterpret_cast<u32x4*>(a_lds + a_chunk_slot(id / CPR_A, id % CPR_A) * 16) = a_stage[it];
    }
#pragma unroll
    for (int it = 0; it < B_IT; ++it) {
      const int id = it * NT + tid;
      *reinterpret_cast<u32x4*>(b_lds + b_chunk_slot(id / CPR_B, id % CPR_B) * 16) = b_stage[it];
    }
  };
  auto compute = [&](int slot) {
    load_frags(af0, bf0, slot, 0);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      if (ks & 1) {
        if (ks + 1 < KS) load_frags(af0, bf0, slot, ks + 1);
        mfma_step(af1, bf1);
      } else {
        if (ks + 1 < KS) load_frags(af1, bf1, slot, ks + 1);
        mfma_step(af0, bf0);
      }
    }
  };
  static_assert(STAGES <= 2, "the VGPR-staged ring is 1 or 2 deep");

  load_global(0);
  store_lds(0);
  __syncthreads();
#if STAGES == 2
  // The loads of tile kt+1 are in flight while tile kt is multiplied; one
  // barrier per K-tile.  The last tile is peeled so that the prefetch is
  // unconditional inside the loop.
  for (int kt = 0; kt < NK - 1; ++kt) {
    const int slot = kt & 1;
    load_global(kt + 1);
    compute(slot);
    store_lds(slot ^ 1);
    __syncthreads();
  }
  compute((NK - 1) & 1);
#else
  for (int kt = 0; kt < NK - 1; ++kt) {
    load_global(kt + 1);
    compute(0);
    __syncthreads();
    store_lds(0);
    __syncthreads();
  }
  compute(0);
#endif
#endif  // DECA_DIRECT
#if DECA_EPI_LDS
  __syncthreads();
#endif

  // ---- epilogue ------------------------------------------------------------------
  // acc[mt][nt][i]: m = wm0 + mt*32 + lane%32,
  //                 n = wn0 + nt*32 + (i/4)*8 + (lane/32)*4 + i%4
#if DECA_EPI_LDS
  {
    constexpr int LD = BN + EPI_PAD;
    elem_t* c_lds = reinterpret_cast<elem_t*>(lds);
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int nt = 0; nt < NTL; ++nt)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          half4 h;
#pragma unroll
          for (int e = 0; e < 4; ++e) h[e] = static_cast<elem_t>(acc[mt][nt][q * 4 + e]);
          const int m = wm0 + mt * 32 + l32;
          const int n = wn0 + nt * 32 + q * 8 + khalf * 4;
          *reinterpret_cast<half4*>(c_lds + m * LD + n) = h;
        }
    __syncthreads();
    constexpr int CPR_C = BN / 8;
    static_assert((BM * CPR_C) % NT == 0, "epilogue coverage");
    elem_t* c_g = C + static_cast<size_t>(bm) * BM * N_ + static_cast<size_t>(bn) * BN;
#pragma unroll
    for (int it = 0; it < BM * CPR_C / NT; ++it) {
      const int id = it * NT + tid;
      const int row = id / CPR_C, c = id % CPR_C;
      const u32x4 v = *reinterpret_cast<const u32x4*>(c_lds + row * LD + c * 8);
      *reinterpret_cast<u32x4*>(c_g + static_cast<size_t>(row) * N_ + c * 8) = v;
    }
  }
#else
  {
    elem_t* c_g = C + (static_cast<size_t>(bm) * BM + wm0 + l32) * N_ +
                    static_cast<size_t>(bn) * BN + wn0 + khalf * 4;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int nt = 0; nt < NTL; ++nt)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          half4 h;
#pragma unroll
          for (int e = 0; e < 4; ++e) h[e] = static_cast<elem_t>(acc[mt][nt][q * 4 + e]);
          *reinterpret_cast<half4*>(c_g + static_cast<size_t>(mt) * 32 * N_ + nt * 32 + q * 8) = h;
        }
  }
#endif
}
