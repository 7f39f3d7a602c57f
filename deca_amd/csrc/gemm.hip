// 16-bit x 16-bit -> fp32-accumulate GEMM, C[M,N] = A[M,K] * B[K,N], all row-major
// float16 (or bfloat16 with DECA_BF16), for gfx950 (MFMA v_mfma_f32_32x32x16_f16 /
// _bf16, or the 16x16x32 forms with DECA_MFMA16).
//
// One code object per (shape, GemmConfig); every DECA_* macro is a compile-time
// constant supplied by kernels/gemm_hip.py, as the reference bakes shape and
// config into each generated kernel (src/kernels/gemm_tir.py:123-156).
//
//   DECA_M/N/K    problem size          DECA_BM/BN/BK  workgroup tile
//   DECA_WM/WN    wave tile             DECA_STAGES    LDS ring depth (see DECA_DIRECT)
//   DECA_RASTER   workgroup rows per rasterisation group; 0: an 8 x 4 sub-block of
//                 tiles per XCD, 8 neighbouring sub-blocks in flight
//   DECA_EPI_LDS  1: stage C through LDS for 16-byte stores
//   DECA_XCD      1: remap workgroup ids so that each of the 8 XCDs (private L2)
//                 owns a contiguous slab of tiles
//   DECA_DIRECT   1: global -> LDS loads that bypass the VGPRs, ring of
//                 DECA_STAGES (2..5) tiles; 0: loads staged through VGPRs one
//                 tile ahead, ring of 1 or 2 tiles
//   DECA_TAIL     R > 0: the last R tiles (the partial last wave of workgroups)
//                 are computed as 4 R quarter tiles of BM/2 x BN/2, by
//                 workgroups of the same size with wave tiles WM/2 x WN/2 and a
//                 ring of DECA_TAIL_STAGES slots
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

// The direct-to-LDS loads below set M0 inside their asm statement and declare it
// clobbered, so that the compiler never assumes an M0 value of its own survives one;
// clang notes that M0 is a reserved register, which is the point.
#pragma clang diagnostic ignored "-Winline-asm"

#ifndef DECA_BM
#error "gemm.hip is a template: define the DECA_* macros"
#endif
#ifndef DECA_MIN_WAVES
#define DECA_MIN_WAVES 1  // waves per SIMD the register allocation must leave room for
#endif
#ifndef DECA_BF16
#define DECA_BF16 0
#endif
#ifndef DECA_TAIL
#define DECA_TAIL 0
#endif

#define M_ DECA_M
#define N_ DECA_N
#define K_ DECA_K
#define BK DECA_BK
// s_waitcnt on the vector-memory counter only (gfx9 encoding: vmcnt in bits
// 3:0 and 15:14, expcnt 6:4 and lgkmcnt 11:8 left at "no wait").
#define DECA_WAIT_VMCNT(n) __builtin_amdgcn_s_waitcnt(((n) & 15) | (((n) >> 4) << 14) | 0x0F70)

#ifndef DECA_MFMA16
#define DECA_MFMA16 0  // 1: v_mfma_f32_16x16x32 tiles instead of 32x32x16
#endif
#ifndef DECA_ACC_AGPR
#define DECA_ACC_AGPR 0  // 16x16x32 body: 1 keeps the accumulators in accumulation registers (MFMAs as inline asm)
#endif
#ifndef DECA_DMA_SPREAD
#define DECA_DMA_SPREAD 0  // 16x16x32 body: MFMA groups of a K-tile over which its global->LDS loads are dealt (0: one burst)
#endif
#ifndef DECA_DMA_FIRST
#define DECA_DMA_FIRST 0  // ... and the number of groups behind the barrier that pass before the first load
#endif
#ifndef DECA_EARLY_GROUPS
#define DECA_EARLY_GROUPS 0  // 16x16x32 body: MFMA groups of a K-tile's last k-step issued before its barrier
#endif
#if DECA_BF16
typedef __bf16 elem_t;
#if DECA_MFMA16
#define DECA_MFMA __builtin_amdgcn_mfma_f32_16x16x32_bf16
#define DECA_MFMA_ASM "v_mfma_f32_16x16x32_bf16"
#else
#define DECA_MFMA __builtin_amdgcn_mfma_f32_32x32x16_bf16
#endif
#else
typedef _Float16 elem_t;
#if DECA_MFMA16
#define DECA_MFMA __builtin_amdgcn_mfma_f32_16x16x32_f16
#define DECA_MFMA_ASM "v_mfma_f32_16x16x32_f16"
#else
#define DECA_MFMA __builtin_amdgcn_mfma_f32_32x32x16_f16
#endif
#endif
typedef elem_t half8 __attribute__((ext_vector_type(8)));
typedef elem_t half4 __attribute__((ext_vector_type(4)));
typedef short short4v __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) short4v* lds_s4_ptr;
typedef const __attribute__((address_space(1))) void* gptr;
typedef __attribute__((address_space(3))) void* lptr;


#define TILE_NS full_tile
#define T_BM DECA_BM
#define T_BN DECA_BN
#define T_WM DECA_WM
#define T_WN DECA_WN
#define T_STAGES DECA_STAGES
#include "gemm_tile.inc"
#undef TILE_NS
#undef T_BM
#undef T_BN
#undef T_WM
#undef T_WN
#undef T_STAGES

#if DECA_TAIL
#define TILE_NS quarter_tile
#define T_BM (DECA_BM / 2)
#define T_BN (DECA_BN / 2)
#define T_WM (DECA_WM / 2)
#define T_WN (DECA_WN / 2)
#define T_STAGES DECA_TAIL_STAGES
#include "gemm_tile.inc"
#undef TILE_NS
#undef T_BM
#undef T_BN
#undef T_WM
#undef T_WN
#undef T_STAGES
static_assert(quarter_tile::NT == full_tile::NT, "both tile shapes use the same workgroup");
#endif

constexpr int GM = full_tile::GM;
constexpr int GN = full_tile::GN;
constexpr int TILES = GM * GN - DECA_TAIL;  // full tiles; the rest are split in four
#if DECA_TAIL
constexpr int LDS_BYTES = full_tile::LDS_BYTES > quarter_tile::LDS_BYTES ? full_tile::LDS_BYTES
                                                                           : quarter_tile::LDS_BYTES;
#else
constexpr int LDS_BYTES = full_tile::LDS_BYTES;
#endif
static_assert(DECA_RASTER == 0 || GM % (DECA_RASTER ? DECA_RASTER : 1) == 0,
              "raster group must divide the workgroup rows");
static_assert(LDS_BYTES <= 160 * 1024, "LDS budget");

extern "C" __global__ void __launch_bounds__(full_tile::NT, DECA_MIN_WAVES)
deca_main(const elem_t* __restrict__ A, const elem_t* __restrict__ B,
          elem_t* __restrict__ C) {
  __shared__ __attribute__((aligned(16))) unsigned char lds[LDS_BYTES];

  // ---- workgroup -> tile mapping --------------------------------------------
  // With DECA_TAIL, workgroups TILES .. TILES + 4 * DECA_TAIL - 1 each take a quarter
  // of one of the last DECA_TAIL tiles of the order below; they start as the full
  // tiles of the last whole wave finish and fill the compute units that a partial
  // wave of full tiles would leave idle.
  int lin = blockIdx.x;
  int quarter = -1;
  int bm, bn;
#if DECA_RASTER == 0
  // Workgroups are dealt round-robin to the 8 XCDs.  Each XCD works on an 8 x 4
  // sub-block of tiles at a time (32 workgroups, one per CU: its L2 fetches 12
  // operand panels for 32 tiles), and the 8 sub-blocks in flight are neighbours:
  // sub-blocks are numbered down two rows of sub-blocks at a time, so that 8
  // consecutive ones form a 16 x 16 block of tiles and the 8 L2s together ask the
  // fabric for only 16 A and 16 B panels per 256 tiles.  The two-row bands are
  // walked back and forth, so that consecutive blocks share their A panels, or at
  // the turn their B panels; an odd last row of sub-blocks is walked on its own.
  static_assert(GM % 8 == 0 && GN % 4 == 0, "8 x 4 sub-blocks of tiles");
  static_assert(TILES % 256 == 0, "whole rounds of 8 sub-blocks (the rest is the tail)");
  static_assert(DECA_XCD, "the block order is an XCD order");
  {
    int sq, within;
    if (DECA_TAIL && lin >= TILES) {
      const int t = lin - TILES;
      quarter = t & 3;
      sq = TILES / 32 + (t >> 7);
      within = (t >> 2) & 31;
    } else {
      const int x = lin & 7, idx = lin >> 3;
      sq = (idx >> 5) * 8 + x;
      within = idx & 31;
    }
    constexpr int NB = GM / 8, NC = GN / 4;  // sub-block rows and columns
    constexpr int PAIR = 2 * NC;              // sub-blocks of a two-row band
    const int band = sq / PAIR;
    int sr, sc;
    if (band < NB / 2) {
      sr = 2 * band + (sq % PAIR & 1);
      sc = (sq % PAIR) >> 1;
    } else {
      sr = NB - 1;
      sc = sq - (NB / 2) * PAIR;
    }
    if (band & 1) sc = NC - 1 - sc;
    bm = sr * 8 + (within & 7);
    bn = sc * 4 + (within >> 3);
  }
#else
  if (DECA_TAIL && lin >= TILES) {
    quarter = (lin - TILES) & 3;
    lin = TILES + ((lin - TILES) >> 2);
  } else {
#if DECA_XCD
    // Workgroups are dealt round-robin to the 8 XCDs; give each XCD a
    // contiguous range of tiles so that its L2 sees a compact set of A rows
    // and B columns.
    static_assert(TILES % 8 == 0, "XCD remap needs a multiple of 8 workgroups");
    lin = (lin & 7) * (TILES / 8) + (lin >> 3);
#endif
  }
  {
    constexpr int GROUP = DECA_RASTER * GN;
    bm = (lin / GROUP) * DECA_RASTER + (lin % GROUP) % DECA_RASTER;
    bn = (lin % GROUP) / DECA_RASTER;
  }
#endif

#if DECA_TAIL
  if (quarter >= 0) {
    quarter_tile::run(A, B, C, bm * 2 + (quarter >> 1), bn * 2 + (quarter & 1), lds);
    return;
  }
#endif
  full_tile::run(A, B, C, bm, bn, lds);
}
