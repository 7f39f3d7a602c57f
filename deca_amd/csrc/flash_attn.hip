// FlashAttention forward, O = softmax(scale * Q K^T [+ causal mask]) V, for gfx950.
// Q, K, V, O are contiguous [B, H, S, D] float16; fp32 scores and accumulators.
//
// One code object per (shape, FAConfig); the DECA_* macros are compile-time
// constants supplied by kernels/flash_attn_hip.py, as the reference bakes shape
// and config into each generated kernel (src/kernels/flash_attn_tir.py:83-137).
//
//   DECA_B/H/SQ/SKV/D   problem          DECA_BR   query rows per workgroup
//   DECA_BC             key/value rows per step
//   DECA_NW             waves per workgroup (each owns BR / NW query rows)
//   DECA_STAGES         K/V LDS ring depth (1, 2 or 3; 3 in the plain loop only: tiles are
//                       requested two steps ahead)
//   DECA_QSMEM          1: the Q tile is staged in LDS once and its fragments are read
//                       again from there in every KV step (flash_attn_tir.py:263-281,
//                       345-348) instead of living in VGPRs for the whole kernel
//   DECA_SWIZZLE        0: K/V/Q rows lie linearly in LDS (no XOR swizzle)
//   DECA_SPREAD         n > 0: the K/V loads of the next tile are dealt over the first n
//                       matrix-instruction groups of a step instead of issued in one burst
//                       behind the barrier (plain ring loops and slot loop)
//   DECA_TRUST          1 (plain ring loops): a tile's exponentials are taken against the
//                       running max as it stands, without looking at the tile's own max
//                       first; a tile that turns out to have outgrown it is done again
//   DECA_CAUSAL         1: key j visible to query i iff j <= i (SQ == SKV)
//   DECA_SCALE          softmax scale
//   DECA_PIPE           1: S^T of the next tile is computed before the softmax of
//                       the current one (two S^T accumulators per wave)
//                       2: as 1, and every matrix instruction of an iteration carries
//                       a fixed share of the iteration's vector work ("slots")
//   DECA_MIN_WAVES      waves per SIMD the register allocation leaves room for
//   DECA_LAZY_TAU       the running max follows a tile's max only when that is more
//                       than this many powers of two above it (0: always)
//
// The problem is computed transposed, which is what makes the two MFMA
// products chain without a layout change on CDNA:
//   S^T = K Q^T   first operand K rows (32 keys x 16 d, ds_read_b128),
//                 second operand Q (32 queries x 16 d, kept in VGPRs);
//                 a lane then holds ONE query column (lane % 32) and 16 key
//                 rows per 32-key block, so the row max / row sum of the online
//                 softmax are in-lane reductions plus one exchange with lane^32
//                 (v_permlane32_swap);
//   O^T = V^T P^T first operand V^T (32 d x 16 keys, transposing
//                 ds_read_b64_tr_b16 of the row-major V tile), second operand
//                 P^T taken straight from the S^T accumulator registers (its
//                 register order is, by construction, the k-packed operand
//                 order once the matching key rows are chosen for V).
// The per-query rescale factor is a per-lane scalar.  K/V tiles arrive by
// global->LDS loads one step ahead (ring of DECA_STAGES slots).
//
// Numerics follow src/kernels/flash_attn_tir.py:379-458: unscaled fp32 S; mask
// value -1e30 on tiles crossing the diagonal only; m' = max(m, rowmax S);
// alpha = exp2((m - m') * sl2); p = exp2(S * sl2 - m' * sl2), sl2 = scale * log2e;
// l = l * alpha + sum p (fp32 p); P = fp16(p) feeds the second product;
// O = O * alpha + P V; final O / l -> fp16.  One departure: m' is taken lazily
// (DECA_LAZY_TAU), which leaves O / l the same quotient with p <= 2^tau
// instead of p <= 1 and makes alpha exactly 1 for almost every tile.
#include <hip/hip_runtime.h>

// The direct-to-LDS loads below set M0 inside their asm statement and declare it
// clobbered, so that the compiler never assumes an M0 value of its own survives one;
// clang notes that M0 is a reserved register, which is the point.
#pragma clang diagnostic ignored "-Winline-asm"
#include <type_traits>
#include <utility>

#ifndef DECA_BR
#error "flash_attn.hip is a template: define the DECA_* macros"
#endif

#define D_ DECA_D
#define BR DECA_BR
#define BC DECA_BC
#define NW DECA_NW
#define STAGES DECA_STAGES
#ifndef DECA_LAZY_TAU
#define DECA_LAZY_TAU 8
#endif
#ifndef DECA_EPI_LDS
#define DECA_EPI_LDS 1
#endif
#ifndef DECA_ROLL
#define DECA_ROLL 0  // plain loop with two LDS stages: 1 keeps a single copy of the step
#endif
#ifndef DECA_QSMEM
#define DECA_QSMEM 0
#endif
#ifndef DECA_SWIZZLE
#define DECA_SWIZZLE 1
#endif
#ifndef DECA_SPREAD
#define DECA_SPREAD 0
#endif
#ifndef DECA_TRUST
#define DECA_TRUST 0
#endif
// In the 16x16x32 form the plain loops take a tile's row sums on the matrix pipe (one more
// product per k-step, with a ones operand: four accumulator registers per query tile), which
// frees the vector ALU of one add per score; l is then the sum of the fp16 P that the second
// product also sees, already reduced over the lanes of a query.  (Not the slot loop, whose
// slots carry the adds, nor the plain steps that finish its causal form: l has one meaning
// per kernel.)  -DDECA_MFMASUM=0 builds the vector-ALU sums instead, for comparisons.
#ifndef DECA_MFMASUM
#define DECA_MFMASUM (DECA_MFMA16 && DECA_PIPE == 0)
#endif
#ifndef DECA_MIN_WAVES
#define DECA_MIN_WAVES 1  // waves per SIMD the register allocation must leave room for
#endif

constexpr int NT = NW * 64;
constexpr int WQ = BR / NW;       // query rows per wave
#ifndef DECA_MFMA16
#define DECA_MFMA16 0  // 1: v_mfma_f32_16x16x32_f16 tiles (plain loop only) instead of 32x32x16
#endif
#if DECA_MFMA16
// 16 x 16 accumulator tiles, k-steps of 32.  A lane holds ONE query column (lane % 16)
// and 4 key rows (4 * (lane / 16) .. +3) per 16-key block; the four 16-lane groups of a
// query are reduced with two row swaps.  P^T for one O^T step (32 keys) is the pair of
// key blocks 2kk, 2kk + 1: operand k-index 8g + i is key 4g + i of block 2kk (i < 4) or
// key 4g + i - 4 of block 2kk + 1, and V^T is read in the same key order.
constexpr int TQ = 16;            // queries per MFMA tile
constexpr int MQ = WQ / 16;       // query tiles per wave
constexpr int KT = BC / 16;       // 16-key blocks per step
constexpr int DK = D_ / 32;       // k-steps of S^T = K Q^T
constexpr int DT = D_ / 16;       // 16-d blocks of O^T
constexpr int KK = BC / 32;       // k-steps of O^T = V^T P^T
constexpr int ACC_N = 4;
constexpr int K_CHUNKS_PER_STEP = 4, V_CHUNKS_PER_BLOCK = 2;
static_assert(DECA_PIPE != 1, "the 16x16x32 form is written for the plain and the slot loop");
static_assert(BC % 32 == 0 && WQ % 16 == 0, "tiles of the 16x16x32 form");
#else
constexpr int TQ = 32;
constexpr int MQ = WQ / 32;       // 32-query MFMA tiles per wave
constexpr int KT = BC / 32;       // 32-key blocks per step (S^T row tiles)
constexpr int DK = D_ / 16;       // k-steps of S^T = K Q^T
constexpr int DT = D_ / 32;       // 32-d blocks of O^T
constexpr int KK = BC / 16;       // k-steps of O^T = V^T P^T
constexpr int ACC_N = 16;
constexpr int K_CHUNKS_PER_STEP = 2, V_CHUNKS_PER_BLOCK = 4;
#endif
constexpr int CPR = D_ / 8;       // 16-byte chunks per K/V row
constexpr int TILE_CHUNKS = BC * CPR;
constexpr int TILE_BYTES = TILE_CHUNKS * 16;
constexpr int KV_IT = TILE_CHUNKS / NT;
constexpr int NKV = DECA_SKV / BC;
constexpr int RING_BYTES = 2 * STAGES * TILE_BYTES;
constexpr int Q_LDS_OFFSET = RING_BYTES;                 // the Q tile follows the K/V ring
constexpr int LDS_BYTES = RING_BYTES + (DECA_QSMEM ? BR * D_ * 2 : 0);
constexpr float LOG2E = 1.4426950408889634f;
constexpr float NEG_INF = -1e30f;
constexpr float SL2 = static_cast<float>(DECA_SCALE) * LOG2E;

static_assert(D_ % 64 == 0 && D_ >= 64, "head dim: a multiple of 64 (flash_attn_tir.py:70-72)");
static_assert(BR % (32 * NW) == 0, "each wave owns a multiple of 32 query rows");
static_assert(BC % 32 == 0, "BC must be a multiple of 32");
static_assert(DECA_SQ % BR == 0 && DECA_SKV % BC == 0, "tiles must divide the sequences");
static_assert(TILE_CHUNKS % NT == 0, "loader coverage");
static_assert(STAGES >= 1 && STAGES <= 3, "K/V ring depth");
static_assert(STAGES < 3 || DECA_PIPE == 0, "three stages: plain loop only");
static_assert(!DECA_TRUST || (DECA_PIPE == 0 && STAGES >= 2), "trust: a form of the plain ring loops");
static_assert(STAGES < 3 || 4 * KV_IT <= 63, "two tile pairs in flight fit the 6-bit counter");
static_assert(!DECA_CAUSAL || DECA_SQ == DECA_SKV, "causal needs S_q == S_kv");
static_assert(LDS_BYTES <= 160 * 1024, "LDS budget");
static_assert(2 * KV_IT <= 63, "vmcnt holds 6 bits");

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef short short4v __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
#if DECA_MFMA16
typedef floatx4 acc_t;
#else
typedef floatx16 acc_t;
#endif
typedef __attribute__((address_space(3))) short4v* lds_s4_ptr;
#if DECA_MFMA16
#define DECA_MFMA __builtin_amdgcn_mfma_f32_16x16x32_f16
#else
#define DECA_MFMA __builtin_amdgcn_mfma_f32_32x32x16_f16
#endif
typedef __attribute__((address_space(3))) void* lptr;

// LDS layouts.  Rows are D * 2 bytes: a multiple of 256 bytes (the bank window) when
// D is a multiple of 128, an odd multiple of 128 bytes otherwise (D = 64, 192, 320 ...).
// K tile [BC][D]: 16-byte chunk c of row r sits at chunk slot c ^ k_swz(r), so that
// 16 consecutive rows at one logical chunk land on the 16 different 16-byte groups of
// the window: when all rows alias, the low four chunk bits are XORed with r % 16; when
// rows r and r + 1 sit in different halves of the window, the low three with
// (r / 2) % 8.  Only the low bits of c change, so the slot stays inside the row for any
// number of chunks that is a multiple of 8.  V tile [BC][D]: chunk c of row r sits at
// c ^ v_swz(r), which puts the 4 key rows that one half of a transposing read touches
// (64 bytes each) onto the 4 different 64-byte groups of the window: when all rows
// alias the group is rotated by r % 4, otherwise rows r and r + 2 are told apart by
// bit 1 of r.
constexpr bool ROWS_ALIAS = CPR % 16 == 0;
constexpr int K_XOR_BITS = ROWS_ALIAS ? 4 : 3;
constexpr int V_XOR_BITS = ROWS_ALIAS ? 2 : 1;  // of the 64-byte group index (chunk bits 2..)
#if !DECA_SWIZZLE
// linear rows: every read of a column of chunks hits the same banks
constexpr int k_swz(int) { return 0; }
constexpr int v_swz(int) { return 0; }
#else
constexpr int k_swz(int row) { return ROWS_ALIAS ? (row & 15) : ((row >> 1) & 7); }
#endif
#if !DECA_SWIZZLE
#elif DECA_MFMA16
// (the two 16-lane blocks of a half-wave read rows r and r + 4 of the same 32-byte column
// range: bit 2 of r moves them to different halves of the 64-byte group)
constexpr int v_swz(int row) {
  return (ROWS_ALIAS ? ((row & 3) << 2) : (((row >> 1) & 1) << 2)) | (((row >> 2) & 1) << 1);
}
#else
constexpr int v_swz(int row) { return ROWS_ALIAS ? ((row & 3) << 2) : (((row >> 1) & 1) << 2); }
#endif
// A read of logical chunk c0 + j (c0 compile-time, j and the swizzle from the lane) is
// "lane base XOR constant, plus constant": the bits of c0 that the swizzle can reach go
// into the XOR, the rest is added.
constexpr unsigned k_xor_const(int c0) { return static_cast<unsigned>(c0 & ((1 << K_XOR_BITS) - 1)) * 16u; }
constexpr unsigned k_add_const(int c0) { return static_cast<unsigned>(c0 >> K_XOR_BITS << K_XOR_BITS) * 16u; }
constexpr unsigned v_xor_const(int c0) { return static_cast<unsigned>(c0 & ((4 << V_XOR_BITS) - 1)) * 16u; }
constexpr unsigned v_add_const(int c0) { return static_cast<unsigned>(c0 >> (2 + V_XOR_BITS) << (2 + V_XOR_BITS)) * 16u; }

// Slices per dispatch group of the causal kernel: the smallest divisor g of the
// slices of an XCD with g * nq >= 32 workgroups (64 when a slice has 16 or more
// query tiles).
constexpr int causal_group(int nq, int bhx) {
  const int want = nq >= 16 ? 64 : 32;
  for (int g = 1; g < bhx; ++g)
    if (bhx % g == 0 && g * nq >= want) return g;
  return bhx;
}

// f(integral_constant<int, 0>) ... f(integral_constant<int, N-1>), in order
template <class F, int... I>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, I...>) {
  (f(std::integral_constant<int, I>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(f, std::make_integer_sequence<int, (N > 0 ? N : 0)>{});
}

// The values of lanes l and l ^ 32 (the two 32-lane halves of the wave hold the two
// halves of a query's keys): v_permlane32_swap on two copies of x leaves the lower
// half's value in every lane of one copy and the upper half's in the other.  A vector
// ALU instruction; the generic cross-lane shuffle would go through the LDS pipe.
__device__ __forceinline__ void both_halves(float x, float& lower, float& upper) {
  typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
  const unsigned u = __builtin_bit_cast(unsigned, x);
  const u32x2 r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  const unsigned lo = r.x, hi = r.y;
  lower = __builtin_bit_cast(float, lo);
  upper = __builtin_bit_cast(float, hi);
}
__device__ __forceinline__ float max_halves(float x) {
  float a, b;
  both_halves(x, a, b);
  return fmaxf(a, b);
}
__device__ __forceinline__ float sum_halves(float x) {
  float a, b;
  both_halves(x, a, b);
  return a + b;
}
// The same for the 16-lane rows l and l ^ 16 (v_permlane16_swap).
__device__ __forceinline__ void both_rows(float x, float& even, float& odd) {
  typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
  const unsigned u = __builtin_bit_cast(unsigned, x);
  const u32x2 r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  const unsigned e = r.x, o = r.y;
  even = __builtin_bit_cast(float, e);
  odd = __builtin_bit_cast(float, o);
}
// Reduction over the lanes that hold one query column: lanes l and l ^ 32 in the 32x32x16
// form, the four lanes l % 16 + {0, 16, 32, 48} in the 16x16x32 form.
__device__ __forceinline__ float max_over_query(float x) {
#if DECA_MFMA16
  float a, b;
  both_rows(x, a, b);
  x = fmaxf(a, b);
#endif
  return max_halves(x);
}
__device__ __forceinline__ float sum_over_query(float x) {
#if DECA_MFMA16
  float a, b;
  both_rows(x, a, b);
  x = a + b;
#endif
  return sum_halves(x);
}

#define DECA_WAIT_VMCNT(n) __builtin_amdgcn_s_waitcnt(((n) & 15) | (((n) >> 4) << 14) | 0x0F70)

extern "C" __global__ void __launch_bounds__(NT, DECA_MIN_WAVES)
deca_main(const _Float16* __restrict__ Q, const _Float16* __restrict__ K,
          const _Float16* __restrict__ V, _Float16* __restrict__ O) {
  __shared__ __attribute__((aligned(16))) unsigned char lds[LDS_BYTES];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  const int l32 = lane & 31;
  const int half = lane >> 5;
  // ---- workgroup -> (batch*head, query tile) ------------------------------------------
  // 1-D grid.  Workgroups are dealt round-robin to the 8 XCDs; the remap gives
  // each XCD whole (batch, head) slices, so that the K/V tiles of a slice are
  // fetched into one L2 only and shared there by all of its query tiles.
  constexpr int NQ = DECA_SQ / BR;
  constexpr int TOTAL = NQ * DECA_B * DECA_H;
#if DECA_CAUSAL
  // Query tiles near the end see the most keys.  They are scheduled first
  // (flash_attn_tir.py:152-156), and first across a group of G (batch, head)
  // slices rather than slice by slice: with the longest workgroups of several
  // slices dispatched before any short one, the short ones fill the gaps and the
  // compute units of an XCD finish together.  G is the smallest group that gives
  // every compute unit of the XCD (32) a workgroup, twice that for long rows; larger
  // groups only spread the K/V working set over more slices than the L2 holds
  // (measured at S = 1024 ... 4096: a few percent lost at either end).
  constexpr int BH = DECA_B * DECA_H;
  int bh, qt;
  if (BH % 8 == 0) {
    constexpr int BHX = BH / 8 > 0 ? BH / 8 : 1;  // slices per XCD
    constexpr int G = causal_group(NQ, BHX);
    static_assert(BHX % G == 0, "groups of whole slices");
    const int idx = blockIdx.x >> 3;
    const int in = idx % (G * NQ);
    bh = (blockIdx.x & 7) * BHX + (idx / (G * NQ)) * G + in % G;
    qt = (NQ - 1) - in / G;
  } else {
    bh = blockIdx.x % BH;
    qt = (NQ - 1) - blockIdx.x / BH;
  }
  const int nkv = ((qt + 1) * BR + BC - 1) / BC;
#else
  int lin = blockIdx.x;
  if (TOTAL % 8 == 0) lin = (lin & 7) * (TOTAL / 8) + (lin >> 3);
  const int bh = lin / NQ;
  const int qt = lin % NQ;
  const int nkv = NKV;
#endif
  const _Float16* q_base = Q + (static_cast<size_t>(bh) * DECA_SQ + qt * BR + wave * WQ) * D_;
  const _Float16* k_base = K + static_cast<size_t>(bh) * DECA_SKV * D_;
  const _Float16* v_base = V + static_cast<size_t>(bh) * DECA_SKV * D_;
  _Float16* o_base = O + (static_cast<size_t>(bh) * DECA_SQ + qt * BR + wave * WQ) * D_;

  // ---- K/V tile loads: global -> LDS, asynchronous ------------------------------
  const unsigned lds_u = static_cast<unsigned>(reinterpret_cast<size_t>((lptr)lds));
  unsigned k_voff[KV_IT], v_voff[KV_IT];
#pragma unroll
  for (int it = 0; it < KV_IT; ++it) {
    const int sidx = it * NT + tid;
    const int row = sidx / CPR, cs = sidx % CPR;
    const int ck = cs ^ k_swz(row);
    const int cv = cs ^ v_swz(row);
    k_voff[it] = static_cast<unsigned>(row * D_ + ck * 8) * 2u;
    v_voff[it] = static_cast<unsigned>(row * D_ + cv * 8) * 2u;
  }
  // Inline assembly keeps the compiler's wait-count insertion from forcing
  // vmcnt(0) before every LDS read; waits are explicit and paired with barriers.
  auto dma16 = [&](const _Float16* origin, unsigned voff, unsigned lds_addr) __attribute__((always_inline)) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                 :
                 : "v"(voff), "s"(origin), "s"(lds_addr)
                 : "memory", "m0");
  };
  auto issue_k = [&](int j, int slot) __attribute__((always_inline)) {
    const _Float16* origin = k_base + static_cast<size_t>(j) * BC * D_;
    const unsigned dst = lds_u + slot * TILE_BYTES + wave_u * 1024;
#pragma unroll
    for (int it = 0; it < KV_IT; ++it) dma16(origin, k_voff[it], dst + it * NT * 16);
  };
  auto issue_v = [&](int j, int slot) __attribute__((always_inline)) {
    const _Float16* origin = v_base + static_cast<size_t>(j) * BC * D_;
    const unsigned dst = lds_u + (STAGES + slot) * TILE_BYTES + wave_u * 1024;
#pragma unroll
    for (int it = 0; it < KV_IT; ++it) dma16(origin, v_voff[it], dst + it * NT * 16);
  };

  // Load number l of the 2 * KV_IT that bring in tile j (K chunks first, then V), and the
  // share of window position i out of n: all waves of a workgroup leave the step's barrier
  // together, and issued in one burst their loads queue up at the CU's one load path (a
  // 64-lane x 16-byte load per 16 clocks) while the waves in that queue issue nothing else.
  auto issue_kv_load = [&](int jk, int kslot, int jv, int vslot, int l) __attribute__((always_inline)) {
    if (l < KV_IT) {
      if (jk < nkv)
        dma16(k_base + static_cast<size_t>(jk) * BC * D_, k_voff[l],
              lds_u + kslot * TILE_BYTES + wave_u * 1024 + l * NT * 16);
    } else {
      dma16(v_base + static_cast<size_t>(jv) * BC * D_, v_voff[l - KV_IT],
            lds_u + (STAGES + vslot) * TILE_BYTES + wave_u * 1024 + (l - KV_IT) * NT * 16);
    }
  };
  auto issue_kv_share = [&](int jk, int kslot, int jv, int vslot, int i, int n) __attribute__((always_inline)) {
#pragma unroll
    for (int l = i * (2 * KV_IT) / n; l < (i + 1) * (2 * KV_IT) / n; ++l)
      issue_kv_load(jk, kslot, jv, vslot, l);
  };

  // ---- Q fragments: VGPR resident for the whole kernel ----------------------------
  // lane (q = lane % 32, half): 8 consecutive d at ks * 16 + half * 8
  // (16x16x32: q = lane % 16, 8 consecutive d at ks * 32 + (lane / 16) * 8)
  const int tb = lane >> 4, ti = lane & 15;
#if DECA_MFMA16
  const int lq = ti;      // query column of this lane inside a query tile
  const int lg = tb;      // which quarter of a k-step / of a key block this lane holds
#else
  const int lq = l32;
  const int lg = half;
#endif
#if DECA_QSMEM
  // The wave's WQ rows of Q go to LDS once, in the K tile's layout (chunk c of row r at
  // slot c ^ k_swz(r)), by the same direct loads as the K/V tiles; the first wait of the
  // loop covers them.  Only this wave reads them back, so no workgroup barrier is owed.
  {
    constexpr int Q_IT = WQ * CPR / 64;
    static_assert((WQ * CPR) % 64 == 0, "a wave's Q rows are whole 1 KiB runs");
    const unsigned dst = lds_u + Q_LDS_OFFSET + wave_u * (WQ * D_ * 2);
    const _Float16* q_origin = Q + (static_cast<size_t>(bh) * DECA_SQ + qt * BR + wave_u * WQ) * D_;
#pragma unroll
    for (int it = 0; it < Q_IT; ++it) {
      const int sidx = it * 64 + lane;
      const int row = sidx / CPR, cs = sidx % CPR;
      dma16(q_origin, static_cast<unsigned>(row * D_ + (cs ^ k_swz(row)) * 8) * 2u, dst + it * 1024);
    }
  }
#else
  half8 qf[MQ][DK];
#pragma unroll
  for (int mq = 0; mq < MQ; ++mq)
#pragma unroll
    for (int ks = 0; ks < DK; ++ks)
      qf[mq][ks] = *reinterpret_cast<const half8*>(
          q_base + (mq * TQ + lq) * D_ + ks * (K_CHUNKS_PER_STEP * 8) + lg * 8);
#endif

  acc_t o_acc[DT][MQ];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int mq = 0; mq < MQ; ++mq)
#pragma unroll
      for (int e = 0; e < ACC_N; ++e) o_acc[dt][mq][e] = 0.0f;
  float m_i[MQ], l_i[MQ];
#pragma unroll
  for (int mq = 0; mq < MQ; ++mq) {
    m_i[mq] = NEG_INF;
    l_i[mq] = 0.0f;
  }

  // ---- LDS read addresses ---------------------------------------------------------------
  // The swizzles only touch address bits that the loop-varying terms (key block,
  // d block, k-step) either leave alone or toggle as a whole, so every read is
  // "per-lane base XOR compile-time constant, plus an immediate offset".
  // K: row = kt*32 + lane%32, chunk = (ks*2 + half) ^ k_swz(row); the row bits used by
  // the swizzle do not depend on kt (k_swz has period 16).
  // (16x16x32: row = kt*16 + lane%16, chunk = (ks*4 + lane/16) ^ k_swz(row))
  unsigned k_lane_base = static_cast<unsigned>(lq * CPR + (lg ^ k_swz(lq))) * 16u;
  auto k_frag_offset = [&](int ks, int kt) __attribute__((always_inline)) {
    return (k_lane_base ^ k_xor_const(ks * K_CHUNKS_PER_STEP)) + k_add_const(ks * K_CHUNKS_PER_STEP) +
           static_cast<unsigned>(kt * TQ * CPR * 16);
  };
  // Q fragment (mq, ks): from the registers, or -- the wave's rows lie in LDS like a K tile
  // whose 32- (16-) row block mq is the query tile -- by the same address as a K fragment.
  auto q_frag = [&](int mq, int ks) __attribute__((always_inline)) -> half8 {
#if DECA_QSMEM
    return *reinterpret_cast<const half8*>(lds + Q_LDS_OFFSET + wave_u * (WQ * D_ * 2) + k_frag_offset(ks, mq));
#else
    return qf[mq][ks];
#endif
  };
  // V: row = kk*16 + r*8 + (half*4 + ti/4), chunk = (dt*4 + tb%2*2 + ti%4/2) ^ v_swz(row)
  // (16x16x32: row = block*16 + (lane/16)*4 + ti/4, chunk = (dt*2 + ti%4/2) ^ v_swz(row))
#if DECA_MFMA16
  const int v_row0 = tb * 4 + (ti >> 2);
  const int v_d0 = 4 * (ti & 3);
#else
  const int v_row0 = (tb >> 1) * 4 + (ti >> 2);
  const int v_d0 = 16 * (tb & 1) + 4 * (ti & 3);
#endif
  const unsigned v_lane_base = static_cast<unsigned>(
      v_row0 * CPR * 16 + (((v_d0 >> 3) ^ v_swz(v_row0)) * 16) +
      ((v_d0 >> 2) & 1) * 8);
  static_assert(CPR >= 8, "D >= 64");
  auto v_frag_offset = [&](int dt, int row0) __attribute__((always_inline)) {
    return (v_lane_base ^ v_xor_const(dt * V_CHUNKS_PER_BLOCK)) + v_add_const(dt * V_CHUNKS_PER_BLOCK) +
           static_cast<unsigned>(row0 * CPR * 16);
  };
  // ---- the three phases of one KV step ----------------------------------------------------
  // S^T = K Q^T for the tile in K slot `kslot`
  auto compute_s = [&](acc_t (&s_acc)[KT][MQ], int kslot, auto&& between) __attribute__((always_inline)) {
    const unsigned char* k_lds = lds + kslot * TILE_BYTES;
#pragma unroll
    for (int kt = 0; kt < KT; ++kt)
#pragma unroll
      for (int mq = 0; mq < MQ; ++mq)
#pragma unroll
        for (int e = 0; e < ACC_N; ++e) s_acc[kt][mq][e] = 0.0f;
#pragma unroll
    for (int ks = 0; ks < DK; ++ks) {
      half8 qk[MQ];
#pragma unroll
      for (int mq = 0; mq < MQ; ++mq) qk[mq] = q_frag(mq, ks);
#pragma unroll
      for (int kt = 0; kt < KT; ++kt) {
        const half8 kf = *reinterpret_cast<const half8*>(k_lds + k_frag_offset(ks, kt));
#pragma unroll
        for (int mq = 0; mq < MQ; ++mq)
          s_acc[kt][mq] = DECA_MFMA(kf, qk[mq], s_acc[kt][mq], 0, 0, 0);
        between(ks * KT + kt);
      }
    }
  };
  auto nothing = [](int) __attribute__((always_inline)) {};
  // Causal mask of tile j.  Only tiles crossing the diagonal need it; every
  // query sees key 0 in tile 0, so its running max is finite before a fully
  // masked block shows up.
  auto mask_s = [&](acc_t (&s_acc)[KT][MQ], int j) __attribute__((always_inline)) {
#if DECA_CAUSAL
    if ((j + 1) * BC - 1 > qt * BR + wave * WQ) {
#pragma unroll
      for (int mq = 0; mq < MQ; ++mq) {
        const int q_idx = qt * BR + wave * WQ + mq * TQ + lq;
#pragma unroll
        for (int kt = 0; kt < KT; ++kt)
#pragma unroll
          for (int e = 0; e < ACC_N; ++e) {
#if DECA_MFMA16
            const int kv_idx = j * BC + kt * 16 + lg * 4 + e;
#else
            const int kv_idx = j * BC + kt * 32 + (e >> 2) * 8 + half * 4 + (e & 3);
#endif
            if (kv_idx > q_idx) s_acc[kt][mq][e] = NEG_INF;
          }
      }
    }
#else
    (void)s_acc;
    (void)j;
#endif
  };
  // The running max only follows the tile's max when that is more than
  // DECA_LAZY_TAU powers of two above it (always for the first tile): until
  // then p = exp2((S - m) * sl2) stays below 2^DECA_LAZY_TAU, which fp16 P and
  // the fp32 sums hold as well as values below 1, and alpha is exactly 1, so
  // the O^T rescale is skipped.  O / l at the end is the same quotient.
  auto lazy_max = [&](float m_old, float mx) __attribute__((always_inline)) {
    const float m_new = fmaxf(m_old, mx);
#if DECA_LAZY_TAU > 0
    return (m_new - m_old) * SL2 > static_cast<float>(DECA_LAZY_TAU) ? m_new : m_old;
#else
    return m_new;
#endif
  };
  // Online softmax of one tile: one query column per lane.  Leaves P^T (fp16,
  // already in operand order) in `pf` and rescales O^T when a running max moved
  // (skipped otherwise: multiplying by 1 is exact).
  auto softmax = [&](acc_t (&s_acc)[KT][MQ], half8 (&pf)[KK][MQ]) __attribute__((always_inline)) {
    float alpha[MQ];
#pragma unroll
    for (int mq = 0; mq < MQ; ++mq) {
      float mx = s_acc[0][mq][0];
#pragma unroll
      for (int kt = 0; kt < KT; ++kt)
#pragma unroll
        for (int e = 0; e < ACC_N; ++e) mx = fmaxf(mx, s_acc[kt][mq][e]);
      mx = max_over_query(mx);
      const float m_new = lazy_max(m_i[mq], mx);
      alpha[mq] = __builtin_amdgcn_exp2f((m_i[mq] - m_new) * SL2);
      m_i[mq] = m_new;
      const float msl = m_new * SL2;
      float sum = 0.0f;
#pragma unroll
      for (int kt = 0; kt < KT; ++kt) {
#pragma unroll
        for (int e = 0; e < ACC_N; ++e) {
          const float p = __builtin_amdgcn_exp2f(__builtin_fmaf(s_acc[kt][mq][e], SL2, -msl));
          s_acc[kt][mq][e] = p;
#if !DECA_MFMASUM
          sum += p;
#endif
        }
#if !DECA_MFMA16
#pragma unroll
        for (int hh = 0; hh < 2; ++hh) {
          half8 h;
#pragma unroll
          for (int e = 0; e < 8; ++e) h[e] = static_cast<_Float16>(s_acc[kt][mq][hh * 8 + e]);
          pf[kt * 2 + hh][mq] = h;
        }
#endif
      }
#if DECA_MFMA16
#pragma unroll
      for (int kk = 0; kk < KK; ++kk) {
        half8 h;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          h[e] = static_cast<_Float16>(s_acc[2 * kk][mq][e]);
          h[4 + e] = static_cast<_Float16>(s_acc[2 * kk + 1][mq][e]);
        }
        pf[kk][mq] = h;
      }
#if DECA_MFMASUM
      {
        half8 ones;
#pragma unroll
        for (int e = 0; e < 8; ++e) ones[e] = (_Float16)1.0f;
        acc_t t;
#pragma unroll
        for (int e = 0; e < ACC_N; ++e) t[e] = 0.0f;
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) t = DECA_MFMA(ones, pf[kk][mq], t, 0, 0, 0);
        sum = t[0];
      }
#endif
#endif
      l_i[mq] = l_i[mq] * alpha[mq] + sum;
    }
    bool moved = false;
#pragma unroll
    for (int mq = 0; mq < MQ; ++mq) moved |= (alpha[mq] != 1.0f);
    if (__builtin_amdgcn_ballot_w64(moved) != 0) {
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int mq = 0; mq < MQ; ++mq)
#pragma unroll
          for (int e = 0; e < ACC_N; ++e) o_acc[dt][mq][e] *= alpha[mq];
    }
  };
#if DECA_TRUST
  // The softmax of a tile taken on trust (`with_max` false): exponentials against the
  // running max as it stands, no max of the tile at all.  A lane's p are then bounded by
  // their own sum (16x16x32 form: by the query's sum over the whole tile, which the matrix
  // pipe delivers), which is looked at afterwards: while no lane of the wave has more than
  // 2^15 in it, every p fits fp16 and the running max may stay (alpha = 1, nothing to
  // rescale); otherwise the call returns true with l and O untouched, and the caller
  // computes S^T again and comes back with `with_max` true, which is `softmax` above.
  // O / l is the same quotient either way.
  auto softmax_flex = [&](acc_t (&s_acc)[KT][MQ], half8 (&pf)[KK][MQ], bool with_max) __attribute__((always_inline)) -> bool {
    float alpha[MQ], tile_sum[MQ];
#pragma unroll
    for (int mq = 0; mq < MQ; ++mq) alpha[mq] = 1.0f;
    if (with_max) {
#pragma unroll
      for (int mq = 0; mq < MQ; ++mq) {
        float mx = s_acc[0][mq][0];
#pragma unroll
        for (int kt = 0; kt < KT; ++kt)
#pragma unroll
          for (int e = 0; e < ACC_N; ++e) mx = fmaxf(mx, s_acc[kt][mq][e]);
        mx = max_over_query(mx);
        const float m_new = lazy_max(m_i[mq], mx);
        alpha[mq] = __builtin_amdgcn_exp2f((m_i[mq] - m_new) * SL2);
        m_i[mq] = m_new;
      }
    }
    bool over = false;
#pragma unroll
    for (int mq = 0; mq < MQ; ++mq) {
      const float msl = m_i[mq] * SL2;
      float sum = 0.0f;
#pragma unroll
      for (int kt = 0; kt < KT; ++kt) {
#pragma unroll
        for (int e = 0; e < ACC_N; ++e) {
          const float p = __builtin_amdgcn_exp2f(__builtin_fmaf(s_acc[kt][mq][e], SL2, -msl));
          s_acc[kt][mq][e] = p;
#if !DECA_MFMASUM
          sum += p;
#endif
        }
#if !DECA_MFMA16
#pragma unroll
        for (int hh = 0; hh < 2; ++hh) {
          half8 h;
#pragma unroll
          for (int e = 0; e < 8; ++e) h[e] = static_cast<_Float16>(s_acc[kt][mq][hh * 8 + e]);
          pf[kt * 2 + hh][mq] = h;
        }
#endif
      }
#if DECA_MFMA16
#pragma unroll
      for (int kk = 0; kk < KK; ++kk) {
        half8 h;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          h[e] = static_cast<_Float16>(s_acc[2 * kk][mq][e]);
          h[4 + e] = static_cast<_Float16>(s_acc[2 * kk + 1][mq][e]);
        }
        pf[kk][mq] = h;
      }
#if DECA_MFMASUM
      {
        // the row sum on the matrix pipe: ones^T P^T has the sum over all keys of the tile
        // in every row of a query's column (already reduced over the lanes of the query)
        half8 ones;
#pragma unroll
        for (int e = 0; e < 8; ++e) ones[e] = (_Float16)1.0f;
        acc_t t;
#pragma unroll
        for (int e = 0; e < ACC_N; ++e) t[e] = 0.0f;
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) t = DECA_MFMA(ones, pf[kk][mq], t, 0, 0, 0);
        sum = t[0];
      }
#endif
#endif
      tile_sum[mq] = sum;
      over |= !(sum <= 32768.0f);  // also true for inf and NaN
    }
    if (!with_max && __builtin_amdgcn_ballot_w64(over) != 0) return true;
#pragma unroll
    for (int mq = 0; mq < MQ; ++mq) l_i[mq] = l_i[mq] * alpha[mq] + tile_sum[mq];
    bool moved = false;
#pragma unroll
    for (int mq = 0; mq < MQ; ++mq) moved |= (alpha[mq] != 1.0f);
    if (__builtin_amdgcn_ballot_w64(moved) != 0) {
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int mq = 0; mq < MQ; ++mq)
#pragma unroll
          for (int e = 0; e < ACC_N; ++e) o_acc[dt][mq][e] *= alpha[mq];
    }
    return false;
  };
#endif
  // O^T += V^T P^T for the tile in V slot `vslot`.  k-slot (half, e) of step kk
  // is key row kk*16 + (e/4)*8 + half*4 + e%4: the order in which the S^T
  // accumulator registers hold the keys.
  auto compute_pv = [&](const half8 (&pf)[KK][MQ], int vslot) __attribute__((always_inline)) {
    const unsigned char* v_lds = lds + (STAGES + vslot) * TILE_BYTES;
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
        half4 h[2];
#pragma unroll
        for (int r = 0; r < 2; ++r) {
#if DECA_MFMA16
          const unsigned char* p = v_lds + v_frag_offset(dt, (2 * kk + r) * 16);
#else
          const unsigned char* p = v_lds + v_frag_offset(dt, kk * 16 + r * 8);
#endif
          h[r] = __builtin_bit_cast(half4, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s4_ptr)(p)));
        }
        const half8 vf = __builtin_shufflevector(h[0], h[1], 0, 1, 2, 3, 4, 5, 6, 7);
#pragma unroll
        for (int mq = 0; mq < MQ; ++mq)
          o_acc[dt][mq] = DECA_MFMA(vf, pf[kk][mq], o_acc[dt][mq], 0, 0, 0);
      }
    }
  };
  auto wait_and_barrier = [&]() __attribute__((always_inline)) {
    DECA_WAIT_VMCNT(0);                  // this lane's outstanding tile loads have landed
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): this wave's LDS reads have returned
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");       // no LDS read of the new tile moves above the barrier
  };

#if STAGES >= 2
  // One KV step.  `slot` is a literal at the call sites of the unrolled loops, so that
  // every LDS address of the step is "lane base + immediate" and needs no address arithmetic.
  auto kv_step = [&](int j, int slot) __attribute__((always_inline)) {
#if STAGES == 3
    // Tiles are requested two steps ahead.  Loads return in order, so tile j has landed
    // for this lane once only the pair of tile j+1 is still outstanding; after the
    // barrier every wave is done with the slot of tile j-1, which tile j+2 takes.
    if (j + 1 < nkv)
      DECA_WAIT_VMCNT(2 * KV_IT);
    else
      DECA_WAIT_VMCNT(0);
    __builtin_amdgcn_s_waitcnt(0xC07F);
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    const int ahead = j + 2;                        // the tile this step requests ...
    const int fill = slot == 0 ? 2 : slot - 1;      // ... and the ring slot it goes to
#else
    // Tile j has landed for every lane, and every wave is done with the slot
    // that tile j+1 is about to overwrite.
    wait_and_barrier();
    const int ahead = j + 1;
    const int fill = slot ^ 1;
#endif
    constexpr int SPREAD_N = DECA_SPREAD < DK * KT ? DECA_SPREAD : DK * KT;
    const bool more = ahead < nkv;
#if DECA_CAUSAL
    // Every key of the tile lies after every query row of this wave (the last tile
    // of a workgroup with BR > BC): all its scores are masked, P = 0 exactly, and
    // there is nothing to add.  (Skipping single masked 32-key blocks of the
    // diagonal tiles as well was tried: the extra code paths cost registers and
    // made the kernel slower.)
    const bool skip = j * BC > qt * BR + wave_u * WQ + WQ - 1;
#else
    const bool skip = false;
#endif
    // one burst behind the barrier, or (DECA_SPREAD) dealt over the S^T groups below
    if (more && (SPREAD_N == 0 || skip)) {
      issue_k(ahead, fill);
      issue_v(ahead, fill);
    }
    if (skip) return;
    acc_t s_acc[KT][MQ];
    half8 pf[KK][MQ];
#if DECA_TRUST
    // The first tile has no running max to trust and takes its own.  Every other tile is
    // taken on trust first; one that outgrew the running max goes round again: S^T is
    // computed once more (p overwrote it; its K tile is still in the slot), then its max.
    bool in_full = j == 0;
#if DECA_CAUSAL
    // a tile that reaches the diagonal for this wave needs the mask: never on trust
    in_full |= (j + 1) * BC - 1 > qt * BR + wave_u * WQ;
#endif
    bool request = more;  // the next tile's loads ride on the first pass only
#pragma unroll 1
    for (;;) {
      // (an opaque copy per pass: the fragment addresses derived from it are then no loop
      // invariants, which the optimiser would compute ahead of the loop and keep in registers)
      asm volatile("" : "+v"(k_lane_base));
#if DECA_SPREAD > 0
      compute_s(s_acc, slot, [&](int i) __attribute__((always_inline)) {
        if (i < SPREAD_N && request) issue_kv_share(ahead, fill, ahead, fill, i, SPREAD_N);
      });
#else
      compute_s(s_acc, slot, nothing);
#endif
      if (in_full) mask_s(s_acc, j);
      if (!softmax_flex(s_acc, pf, in_full)) break;
      in_full = true;
      request = false;
    }
#else
#if DECA_SPREAD > 0
    // the requested tile's loads ride on the first SPREAD_N groups of S^T instructions
    compute_s(s_acc, slot, [&](int i) __attribute__((always_inline)) {
      if (i < SPREAD_N && more) issue_kv_share(ahead, fill, ahead, fill, i, SPREAD_N);
    });
#else
    compute_s(s_acc, slot, nothing);
#endif
    mask_s(s_acc, j);
    softmax(s_acc, pf);
#endif
    compute_pv(pf, slot);
  };
#endif

#if DECA_PIPE
  // ---- software-pipelined loop ------------------------------------------------------------
  // S^T of tile j+1 is computed in the same straight-line block as the
  // exponentials and the second product of tile j, so that one wave's matrix
  // work overlaps its own vector work.  The row statistics (max, rescale factor)
  // of a tile are taken as soon as its S^T is complete, one iteration before its
  // exponentials, which moves the data-dependent O^T rescale (a branch) to the
  // top of the iteration and leaves the rest branch-free.
  // Iteration j needs K_{j+1} and V_j in LDS; both were requested during
  // iteration j-1.  K tile t and V tile t live in slot t % 2 of their rings.
  static_assert(STAGES == 2, "the pipelined loop uses two K and two V slots");
  float alpha[MQ], msl[MQ];
  // m' = max(m, rowmax S); alpha = exp2((m - m') * sl2); msl = m' * sl2
  auto row_stats = [&](const acc_t (&s_acc)[KT][MQ]) __attribute__((always_inline)) {
#pragma unroll
    for (int mq = 0; mq < MQ; ++mq) {
      float mx = s_acc[0][mq][0];
#pragma unroll
      for (int kt = 0; kt < KT; ++kt)
#pragma unroll
        for (int e = 0; e < ACC_N; ++e) mx = fmaxf(mx, s_acc[kt][mq][e]);
      mx = max_over_query(mx);
      const float m_new = lazy_max(m_i[mq], mx);
      alpha[mq] = __builtin_amdgcn_exp2f((m_i[mq] - m_new) * SL2);
      m_i[mq] = m_new;
      msl[mq] = m_new * SL2;
    }
  };
  auto rescale_o = [&]() __attribute__((always_inline)) {
    bool moved = false;
#pragma unroll
    for (int mq = 0; mq < MQ; ++mq) moved |= (alpha[mq] != 1.0f);
    if (__builtin_amdgcn_ballot_w64(moved) != 0) {
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int mq = 0; mq < MQ; ++mq)
#pragma unroll
          for (int e = 0; e < ACC_N; ++e) o_acc[dt][mq][e] *= alpha[mq];
    }
  };
  // p = exp2(S * sl2 - msl); l = l * alpha + sum p; P = fp16(p) in operand order: score
  // number n = kt * ACC_N + e of a lane is element n % 8 of the operand of k-step n / 8
  auto exp_and_pack = [&](acc_t (&s_acc)[KT][MQ], half8 (&pf)[KK][MQ]) __attribute__((always_inline)) {
#pragma unroll
    for (int mq = 0; mq < MQ; ++mq) {
      float sum = 0.0f;
#pragma unroll
      for (int kt = 0; kt < KT; ++kt)
#pragma unroll
        for (int e = 0; e < ACC_N; ++e) {
          const float p = __builtin_amdgcn_exp2f(__builtin_fmaf(s_acc[kt][mq][e], SL2, -msl[mq]));
          s_acc[kt][mq][e] = p;
          sum += p;
        }
#pragma unroll
      for (int kk = 0; kk < KK; ++kk) {
        half8 h;
#pragma unroll
        for (int e = 0; e < 8; ++e)
          h[e] = static_cast<_Float16>(s_acc[(kk * 8 + e) / ACC_N][mq][(kk * 8 + e) % ACC_N]);
        pf[kk][mq] = h;
      }
      l_i[mq] = l_i[mq] * alpha[mq] + sum;
    }
  };
  // S^T of the next tile (K slot `kslot`) fused with the exponentials of the
  // current one: after the MFMAs of step (ks, kt) a fixed share of the current
  // tile's scores is exponentiated, and nothing is allowed to move across the
  // step boundary, so the matrix pipe and the vector ALU stay busy together.
#if DECA_PIPE == 1
  auto s_next_and_exp = [&](floatx16 (&s_nxt)[KT][MQ], floatx16 (&s_cur)[KT][MQ],
                            half8 (&pf)[KK][MQ], int kslot) {
    const unsigned char* k_lds = lds + kslot * TILE_BYTES;
    constexpr int STEPS = DK * KT;
    constexpr int NE_ = KT * 16;  // scores of the current tile per lane and q tile, dealt over the steps
    const floatx16 zero = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f,
                           0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
    float sum[MQ];
#pragma unroll
    for (int mq = 0; mq < MQ; ++mq) sum[mq] = 0.0f;
    half8 kf_next = *reinterpret_cast<const half8*>(k_lds + k_lane_base);
#pragma unroll
    for (int step = 0; step < STEPS; ++step) {
      const int ks = step / KT, kt = step % KT;
      const half8 kf = kf_next;
      if (step + 1 < STEPS) {
        const int ks1 = (step + 1) / KT, kt1 = (step + 1) % KT;
        kf_next = *reinterpret_cast<const half8*>(k_lds + k_frag_offset(ks1, kt1));
      }
#pragma unroll
      for (int mq = 0; mq < MQ; ++mq)
        s_nxt[kt][mq] = __builtin_amdgcn_mfma_f32_32x32x16_f16(
            kf, q_frag(mq, ks), ks == 0 ? zero : s_nxt[kt][mq], 0, 0, 0);
#pragma unroll
      for (int mq = 0; mq < MQ; ++mq)
#pragma unroll
        for (int lin = step * NE_ / STEPS; lin < (step + 1) * NE_ / STEPS; ++lin) {
          const int ct = lin / 16, ce = lin % 16;
          const float p =
              __builtin_amdgcn_exp2f(__builtin_fmaf(s_cur[ct][mq][ce], SL2, -msl[mq]));
          s_cur[ct][mq][ce] = p;
          sum[mq] += p;
          if (lin % 8 == 7) {  // an 8-key block is complete: pack it in operand order
            half8 h;
#pragma unroll
            for (int e = 0; e < 8; ++e)
              h[e] = static_cast<_Float16>(s_cur[ct][mq][(ce / 8) * 8 + e]);
            pf[ct * 2 + ce / 8][mq] = h;
          }
        }
      __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int mq = 0; mq < MQ; ++mq) l_i[mq] = l_i[mq] * alpha[mq] + sum[mq];
  };
#endif

#if DECA_PIPE == 2
  // ---- slot-interleaved loop ----------------------------------------------------------------
  // One iteration = NS slots, one matrix instruction (per query tile) each: first
  // the S^T of tile j+1, then O^T += V_j^T P_j^T.  Every slot also carries a fixed
  // share of the vector work, so that the vector ALU runs in the shadow of the
  // matrix pipe instead of in a phase of its own: the exponentials of tile j in
  // three skewed stages (scale-and-shift in slot t-1, exp2 in slot t, row sum and
  // fp16 packing in slot t+1; they run ahead of the O^T slots that consume them),
  // and the running max of tile j+1 (O^T slots).
  // Nothing moves across a slot boundary; operand fragments are read from LDS two
  // slots ahead.
  static_assert(STAGES == 2, "two K and two V slots");
  static_assert(KT % 2 == 0, "S^T chains are issued in pairs");
  constexpr int S_SLOTS = KT * DK, PV_SLOTS = KK * DT, NS = S_SLOTS + PV_SLOTS;
  constexpr int NE = KT * ACC_N;          // scores per lane and query tile
  constexpr int NM = NE / 2;              // max3 operations of the running max
  constexpr int PVM = PV_SLOTS - 1;       // O^T slots that carry the running max
  struct Sched {
    static constexpr int ne_s() { return NE * 5 / 8; }          // exponentials under the S^T slots
    static constexpr int pve() { return PV_SLOTS - DT - 2; }    // O^T slots carrying the rest
    // scores exponentiated by the end of slot t
    static constexpr int e_end(int t) {
      if (t < 0) return 0;
      if (t < S_SLOTS) return ((t + 1) * ne_s()) / S_SLOTS;
      const int v = ne_s() + ((t - S_SLOTS + 1) * (NE - ne_s()) + pve() - 1) / pve();
      return v < NE ? v : NE;
    }
    // the 8 scores of k-step kk are packed one slot after their exp2 and must be
    // there before the first O^T slot of that k-step
    static constexpr bool ok() {
      if (pve() < 1) return false;
      for (int kk = 0; kk < KK; ++kk)
        if (e_end(S_SLOTS + kk * DT - 2) < 8 * (kk + 1)) return false;
      return e_end(NS - 3) == NE;
    }
  };
  static_assert(Sched::ok(), "the exponentials do not meet the O^T slots in time");
  auto finish_stats = [&](float (&mx)[MQ]) __attribute__((always_inline)) {
#pragma unroll
    for (int mq = 0; mq < MQ; ++mq) {
      const float mxx = max_over_query(mx[mq]);
      const float m_new = lazy_max(m_i[mq], mxx);
      alpha[mq] = __builtin_amdgcn_exp2f((m_i[mq] - m_new) * SL2);
      m_i[mq] = m_new;
      msl[mq] = m_new * SL2;
    }
  };
  half2v pf2[KK][MQ][4];
  // Score number n of a lane and query tile lives in accumulator n / ACC_N, register n % ACC_N.
  auto fused = [&](auto v_slot, acc_t (&sc)[KT][MQ], acc_t (&sn)[KT][MQ], int j) __attribute__((always_inline)) {
    constexpr int VSLOT = decltype(v_slot)::value;  // V_j; K_{j+1} is in the other K slot
    const unsigned char* k_lds = lds + (VSLOT ^ 1) * TILE_BYTES;
    const unsigned char* v_lds = lds + (STAGES + VSLOT) * TILE_BYTES;
    acc_t zero;
#pragma unroll
    for (int e = 0; e < ACC_N; ++e) zero[e] = 0.0f;
    // slot t < S_SLOTS: pair p of key blocks, k-step ks, block kt; else k-step kk, d block dt
    auto read_frag = [&](auto tc) __attribute__((always_inline)) -> half8 {
      constexpr int t = decltype(tc)::value;
      if constexpr (t < S_SLOTS) {
        constexpr int pr = t / (2 * DK), r = t % (2 * DK), ks = r / 2, kt = 2 * pr + r % 2;
        return *reinterpret_cast<const half8*>(k_lds + k_frag_offset(ks, kt));
      } else {
        constexpr int u = t - S_SLOTS, kk = u / DT, dt = u % DT;
        constexpr int V_ROW_STEP = DECA_MFMA16 ? 16 : 8;  // the two key quartets of a lane
        const half4 h0 = __builtin_bit_cast(half4, __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (lds_s4_ptr)(v_lds + v_frag_offset(dt, kk * 2 * V_ROW_STEP))));
        const half4 h1 = __builtin_bit_cast(half4, __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (lds_s4_ptr)(v_lds + v_frag_offset(dt, kk * 2 * V_ROW_STEP + V_ROW_STEP))));
        return __builtin_shufflevector(h0, h1, 0, 1, 2, 3, 4, 5, 6, 7);
      }
    };
    float sum[MQ][2], mx[MQ];
#pragma unroll
    for (int mq = 0; mq < MQ; ++mq) sum[mq][0] = sum[mq][1] = 0.0f;
    // An empty asm that reads and writes a register: the value has to exist at this
    // point, which keeps the optimiser from sinking the operation that produces it
    // out of its slot, towards its first real use.
    auto pin = [](auto& v) { asm volatile("" : "+v"(v)); };
    // the vector work of slot t (t = -1: the scale-and-shift that slot 0 needs)
    auto valu = [&](auto tc) __attribute__((always_inline)) {
      constexpr int t = decltype(tc)::value;
      // (compile-time loops over the query tiles: an unrolling pragma gives up on
      // bodies of this size, and the accumulators would land in scratch memory)
      static_for<MQ>([&](auto mqc) {
        constexpr int mq = decltype(mqc)::value;
        // row sum and packing of what slot t-1 exponentiated
        static_for<Sched::e_end(t - 1) - Sched::e_end(t - 2)>([&](auto ic) {
          constexpr int e = Sched::e_end(t - 2) + decltype(ic)::value;
          sum[mq][e & 1] += sc[e / ACC_N][mq][e % ACC_N];
          pin(sum[mq][e & 1]);
          if constexpr (e & 1) {
            typedef float float2v __attribute__((ext_vector_type(2)));
            const float2v pr = {sc[e / ACC_N][mq][e % ACC_N - 1], sc[e / ACC_N][mq][e % ACC_N]};
            unsigned packed = __builtin_bit_cast(unsigned, __builtin_convertvector(pr, half2v));
            pin(packed);
            pf2[e / 8][mq][(e % 8) / 2] = __builtin_bit_cast(half2v, packed);
          }
        });
        static_for<Sched::e_end(t) - Sched::e_end(t - 1)>([&](auto ic) {
          constexpr int e = Sched::e_end(t - 1) + decltype(ic)::value;
          sc[e / ACC_N][mq][e % ACC_N] = __builtin_amdgcn_exp2f(sc[e / ACC_N][mq][e % ACC_N]);
        });
        static_for<Sched::e_end(t + 1) - Sched::e_end(t)>([&](auto ic) {
          constexpr int e = Sched::e_end(t) + decltype(ic)::value;
          sc[e / ACC_N][mq][e % ACC_N] = __builtin_fmaf(sc[e / ACC_N][mq][e % ACC_N], SL2, -msl[mq]);
        });
        if constexpr (t >= S_SLOTS && t - S_SLOTS < PVM) {
          constexpr int u = t - S_SLOTS;
          if constexpr (u == 0) mx[mq] = sn[0][mq][0];
          constexpr int lo = (u * NM) / PVM, hi = ((u + 1) * NM) / PVM;
          static_for<hi - lo>([&](auto ic) {
            constexpr int i = lo + decltype(ic)::value;
            mx[mq] = fmaxf(fmaxf(mx[mq], sn[2 * i / ACC_N][mq][2 * i % ACC_N]),
                           sn[2 * i / ACC_N][mq][2 * i % ACC_N + 1]);
            pin(mx[mq]);
          });
        }
      });
    };
    half8 frag[3];
    frag[0] = read_frag(std::integral_constant<int, 0>{});
    frag[1] = read_frag(std::integral_constant<int, 1>{});
    valu(std::integral_constant<int, -1>{});
    __builtin_amdgcn_sched_barrier(0);
    static_for<NS>([&](auto tc) {
      constexpr int t = decltype(tc)::value;
      if constexpr (t + 2 < NS) frag[(t + 2) % 3] = read_frag(std::integral_constant<int, t + 2>{});
      // K_{j+2} and V_{j+1} go where K_j and V_{j-1} were: their loads ride on the first slots
      constexpr int SPREAD_S = DECA_SPREAD < NS ? DECA_SPREAD : NS;
      if constexpr (t < SPREAD_S) issue_kv_share(j + 2, VSLOT, j + 1, VSLOT ^ 1, t, SPREAD_S);
      if constexpr (t < S_SLOTS) {
        constexpr int pr = t / (2 * DK), r = t % (2 * DK), ks = r / 2, kt = 2 * pr + r % 2;
        static_for<MQ>([&](auto mqc) {
          constexpr int mq = decltype(mqc)::value;
          sn[kt][mq] = DECA_MFMA(frag[t % 3], q_frag(mq, ks), ks == 0 ? zero : sn[kt][mq], 0, 0, 0);
        });
      } else {
        constexpr int u = t - S_SLOTS, kk = u / DT, dt = u % DT;
        static_for<MQ>([&](auto mqc) {
          constexpr int mq = decltype(mqc)::value;
          const half8 pfr = __builtin_shufflevector(
              __builtin_shufflevector(pf2[kk][mq][0], pf2[kk][mq][1], 0, 1, 2, 3),
              __builtin_shufflevector(pf2[kk][mq][2], pf2[kk][mq][3], 0, 1, 2, 3), 0, 1, 2, 3, 4, 5, 6, 7);
          o_acc[dt][mq] = DECA_MFMA(frag[t % 3], pfr, o_acc[dt][mq], 0, 0, 0);
        });
      }
      valu(tc);
      __builtin_amdgcn_sched_barrier(0);
    });
#pragma unroll
    for (int mq = 0; mq < MQ; ++mq) l_i[mq] = l_i[mq] * alpha[mq] + (sum[mq][0] + sum[mq][1]);
    finish_stats(mx);
  };
  half8 pf[KK][MQ];
  // tile j: softmax and second product; tile j+1: first product and row statistics
  auto step = [&](auto cur_slot, acc_t (&sc)[KT][MQ], acc_t (&sn)[KT][MQ], int j) __attribute__((always_inline)) {
    constexpr int cur = decltype(cur_slot)::value;  // == j % 2
    wait_and_barrier();  // K_{j+1}, V_j landed; everyone is done with K_j and V_{j-1}
#if DECA_SPREAD == 0
    if (j + 2 < nkv) issue_k(j + 2, cur);
    issue_v(j + 1, cur ^ 1);
#endif
    // The O^T rescale stays out of the slots: with the lazy running max it is needed
    // for the first tile and then hardly ever, so it is a branch of its own here.
    rescale_o();
    fused(cur_slot, sc, sn, j);
  };
  auto tail = [&](acc_t (&sc)[KT][MQ], int j) __attribute__((always_inline)) {
    wait_and_barrier();
#if DECA_CAUSAL
    // the diagonal tiles follow: V_{j+1} goes where V_{j-1} was (K_{j+1} is under way)
    issue_v(j + 1, (j + 1) & 1);
#endif
    rescale_o();
    exp_and_pack(sc, pf);
    compute_pv(pf, j & 1);
  };
  const std::integral_constant<int, 0> even;
  const std::integral_constant<int, 1> odd;
#if DECA_CAUSAL
  // Two phases.  The nd tiles that lie below the diagonal for every row of the
  // workgroup need no mask: they run through the slot loop.  The tiles that reach
  // the diagonal follow as plain steps (S^T, mask, softmax, O^T one after the
  // other), which keeps a second, mask-aware copy of the slot sequence out of the
  // register allocation.
  const int nd = (qt * BR) / BC;
  int j0 = 0;
  issue_k(0, 0);
  issue_v(0, 0);
  if (nd >= 2) {
    issue_k(1, 1);
    acc_t s_a[KT][MQ], s_b[KT][MQ];
    wait_and_barrier();
    compute_s(s_a, 0, nothing);
    row_stats(s_a);
    int j = 0;
    for (; j + 2 < nd; j += 2) {
      step(even, s_a, s_b, j);
      step(odd, s_b, s_a, j + 1);
    }
    if (j + 1 < nd) {
      step(even, s_a, s_b, j);
      tail(s_b, j + 1);
    } else {
      tail(s_a, j);
    }
    j0 = nd;
  }
  if (j0 & 1) {
    kv_step(j0, 1);
    ++j0;
  }
  for (int j = j0; j < nkv; j += 2) {
    kv_step(j, 0);
    if (j + 1 < nkv) kv_step(j + 1, 1);
  }
#else
  issue_k(0, 0);
  issue_v(0, 0);
  if (nkv > 1) issue_k(1, 1);
  acc_t s_a[KT][MQ], s_b[KT][MQ];
  wait_and_barrier();
  compute_s(s_a, 0, nothing);
  row_stats(s_a);
  {
    int j = 0;
    for (; j + 2 < nkv; j += 2) {
      step(even, s_a, s_b, j);
      step(odd, s_b, s_a, j + 1);
    }
    if (j + 1 < nkv) {
      step(even, s_a, s_b, j);
      tail(s_b, j + 1);
    } else {
      tail(s_a, j);
    }
  }
#endif
#else
  issue_k(0, 0);
  issue_v(0, 0);
  if (nkv > 1) issue_k(1, 1);
  floatx16 s_cur[KT][MQ], s_nxt[KT][MQ];
  half8 pf[KK][MQ];
  wait_and_barrier();
  compute_s(s_cur, 0, nothing);
  mask_s(s_cur, 0);
  row_stats(s_cur);
  for (int j = 0; j < nkv - 1; ++j) {
    const int cur = j & 1;
    wait_and_barrier();  // K_{j+1}, V_j landed; everyone is done with K_j and V_{j-1}
    if (j + 2 < nkv) issue_k(j + 2, cur);
    issue_v(j + 1, cur ^ 1);
    rescale_o();
    // -- matrix and vector work of two different tiles, interleaved step by step --
    s_next_and_exp(s_nxt, s_cur, pf, cur ^ 1);
    compute_pv(pf, cur);
    mask_s(s_nxt, j + 1);
    row_stats(s_nxt);
#pragma unroll
    for (int kt = 0; kt < KT; ++kt)
#pragma unroll
      for (int mq = 0; mq < MQ; ++mq) s_cur[kt][mq] = s_nxt[kt][mq];
  }
  // last tile: nothing left to prefetch
  wait_and_barrier();
#if DECA_CAUSAL
  // (unless every key of it lies after every query row of this wave: P = 0 exactly)
  if ((nkv - 1) * BC <= qt * BR + wave_u * WQ + WQ - 1)
#endif
  {
    rescale_o();
    exp_and_pack(s_cur, pf);
    compute_pv(pf, (nkv - 1) & 1);
  }
#endif
#else
  issue_k(0, 0);
  issue_v(0, 0);
#if STAGES == 3
  if (nkv > 1) {
    issue_k(1, 1);
    issue_v(1, 1);
  }
#if DECA_ROLL
#pragma unroll 1
  for (int j = 0, slot = 0; j < nkv; ++j, slot = slot == 2 ? 0 : slot + 1) kv_step(j, slot);
#else
  for (int j = 0; j < nkv; j += 3) {
    kv_step(j, 0);
    if (j + 1 < nkv) kv_step(j + 1, 1);
    if (j + 2 < nkv) kv_step(j + 2, 2);
  }
#endif
#elif STAGES == 2 && DECA_ROLL
  // one copy of the step, the ring slot a run-time value
#pragma unroll 1
  for (int j = 0; j < nkv; ++j) kv_step(j, j & 1);
#elif STAGES == 2
  for (int j = 0; j < nkv; j += 2) {
    kv_step(j, 0);
    if (j + 1 < nkv) kv_step(j + 1, 1);
  }
#else
  for (int j = 0; j < nkv; ++j) {
    wait_and_barrier();
    acc_t s_acc[KT][MQ];
    half8 pf[KK][MQ];
    compute_s(s_acc, 0, nothing);
    mask_s(s_acc, j);
    softmax(s_acc, pf);
    compute_pv(pf, 0);
    // single slot: everyone must be done reading before the refill
    __builtin_amdgcn_s_waitcnt(0xC07F);
    __builtin_amdgcn_s_barrier();
    if (j + 1 < nkv) {
      issue_k(j + 1, 0);
      issue_v(j + 1, 0);
    }
  }
#endif
#endif

  // ---- epilogue: O[q][d] = O^T[d][q] / l ----------------------------------------------
  // o_acc[dt][mq][e]: q = mq*32 + lane%32, d = dt*32 + (e/4)*8 + half*4 + e%4.
  // A lane owns 8-byte pieces of a row; when the K/V ring is large enough the
  // wave's [WQ][D] tile is staged through it (rows padded by 8 halves to spread
  // the banks) and written with 16-byte stores that cover whole rows.
  constexpr int EPI_LD = D_ + 8;
  constexpr bool EPI_LDS = DECA_EPI_LDS && LDS_BYTES >= BR * EPI_LD * 2;
  typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
  if (EPI_LDS) {
    __builtin_amdgcn_s_waitcnt(0xC07F);
    __builtin_amdgcn_s_barrier();  // every wave is done reading K/V tiles
  }
  _Float16* o_lds = reinterpret_cast<_Float16*>(lds) + wave * WQ * EPI_LD;
#pragma unroll
  for (int mq = 0; mq < MQ; ++mq) {
#if DECA_MFMASUM
    const float l = l_i[mq];  // the matrix pipe's sums are already over all lanes of the query
#else
    const float l = sum_over_query(l_i[mq]);
#endif
    const float inv = 1.0f / l;
    // (16x16x32: o_acc[dt][mq][e]: q = mq*16 + lane%16, d = dt*16 + (lane/16)*4 + e)
    _Float16* o_row = EPI_LDS ? o_lds + (mq * TQ + lq) * EPI_LD + lg * 4
                              : o_base + (mq * TQ + lq) * D_ + lg * 4;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int g = 0; g < ACC_N / 4; ++g) {
        half4 h;
#pragma unroll
        for (int e = 0; e < 4; ++e) h[e] = static_cast<_Float16>(o_acc[dt][mq][g * 4 + e] * inv);
        *reinterpret_cast<half4*>(o_row + dt * TQ + g * 8) = h;
      }
  }
  if (EPI_LDS) {
    // the tile is private to the wave: its own LDS writes only need to have landed
    __builtin_amdgcn_s_waitcnt(0xC07F);
    __builtin_amdgcn_wave_barrier();
    constexpr int CHUNKS = WQ * CPR;  // 16-byte chunks of the wave's tile
#pragma unroll
    for (int it = 0; it < CHUNKS / 64; ++it) {
      const int idx = it * 64 + lane;
      const int row = idx / CPR, c = idx % CPR;
      const u32x4 v = *reinterpret_cast<const u32x4*>(o_lds + row * EPI_LD + c * 8);
      *reinterpret_cast<u32x4*>(o_base + row * D_ + c * 8) = v;
    }
  }
}
