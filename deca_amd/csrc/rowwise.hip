// Row-wise softmax / RMSNorm over an [M, N] row-major 16-bit tensor, gfx950.
//
// One code object per (op, shape, dtype, config): every DECA_* macro below is
// a compile-time constant supplied by kernels/rowwise_hip.py, as the reference
// bakes shape and RowConfig into each generated kernel
// (src/kernels/rowwise_tir.py:99-127).
//
//   DECA_OP      0 softmax, 1 rmsnorm
//   DECA_M/N     rows / reduced dimension
//   DECA_BF16    0 float16, 1 bfloat16
//   DECA_TPR     lanes cooperating on one row (16, 32, 64, ... 1024)
//   DECA_RPB     rows per workgroup
//   DECA_VEC     elements per vector access (8 -> 16 B, 4 -> 8 B)
//   DECA_MODE    0 reg (row cached in VGPRs), 1 twopass (row streamed twice)
//   DECA_UNROLL  chunks in flight per twopass iteration
//   DECA_HINT    1: non-temporal loads of read-once data and non-temporal stores
//   DECA_LEAN    1 (reg mode): nothing but the packed row stays in registers between
//                the reduction and the stores -- the fp32 values are computed again
//   DECA_EPS     RMSNorm epsilon
//
// Lane t of a row owns the VEC-element chunks (c * TPR + t) * VEC, so one wave
// touches 64 * VEC * 2 contiguous bytes per access (1 KiB at VEC = 8).
// Reductions: DPP butterflies inside a wave (quad_perm, row_half_mirror,
// row_mirror), v_permlane16_swap / v_permlane32_swap across the 16- and 32-lane
// halves (register exchanges, no LDS pipe), then an LDS exchange between the waves
// of a row.  All math is fp32.
//
// Numerics follow src/kernels/rowwise_tir.py:278-389:
//   softmax: m2 = max(x) * log2e; y = exp2(x * log2e - m2) * (1 / sum)
//   rmsnorm: r = rsqrt(sum(x^2) / N + eps); y = dtype(f32(dtype(x * r)) * f32(w))
#include <hip/hip_runtime.h>

#ifndef DECA_OP
#error "rowwise.hip is a template: define the DECA_* macros"
#endif

#define TPR DECA_TPR
#define RPB DECA_RPB
#define VEC DECA_VEC
#define NT (TPR * RPB)
#define SPAN (TPR * VEC)
#define NCHUNK ((DECA_N + SPAN - 1) / SPAN)
#define C_FULL (DECA_N / SPAN)
#define RED_LANES (TPR < 64 ? TPR : 64)
#define NW (TPR / 64 > 0 ? TPR / 64 : 1)

static_assert(DECA_N % VEC == 0, "N must be a multiple of the vector width");
static_assert(DECA_M % RPB == 0, "M must be a multiple of rows_per_block");
static_assert(NT % 64 == 0 && NT <= 1024, "workgroup must be whole waves");
static_assert(VEC == 8 || VEC == 4 || VEC == 2, "vec");

#if DECA_BF16
typedef __bf16 elem_t;
#else
typedef _Float16 elem_t;
#endif
typedef elem_t vec_t __attribute__((ext_vector_type(VEC)));

#ifndef DECA_LEAN
#define DECA_LEAN 0
#endif

#define LOG2E 1.4426950408889634f
#define NEG_INF (-1e30f)

// ---------------------------------------------------------------------------
// cross-lane helpers
// ---------------------------------------------------------------------------
template <int CTRL>
__device__ __forceinline__ float dpp_f(float v) {
  int r = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true);
  return __builtin_bit_cast(float, r);
}

struct MaxOp {
  __device__ __forceinline__ float operator()(float a, float b) const { return fmaxf(a, b); }
};
struct AddOp {
  __device__ __forceinline__ float operator()(float a, float b) const { return a + b; }
};

// All-reduce over groups of LANES consecutive lanes of a wave64.  Steps 4 and 8
// use mirrors instead of xor: every quad (then every 8 lanes) already holds one
// value, so the mirrored partner supplies the other half's value.
template <int LANES, class Op>
__device__ __forceinline__ float wave_allreduce(float v, Op op) {
  if (LANES >= 2) v = op(v, dpp_f<0xB1>(v));   // quad_perm [1,0,3,2]
  if (LANES >= 4) v = op(v, dpp_f<0x4E>(v));   // quad_perm [2,3,0,1]
  if (LANES >= 8) v = op(v, dpp_f<0x141>(v));  // row_half_mirror
  if (LANES >= 16) v = op(v, dpp_f<0x140>(v)); // row_mirror
  // The last two steps pair 16-lane rows, then the 32-lane halves, with the row
  // swaps of gfx950 (v_permlane16_swap / v_permlane32_swap on two copies of v:
  // one copy ends up with the even rows' values in both rows of a pair, the other
  // with the odd rows'), which stay in the vector ALU instead of going through LDS.
  typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
  if (LANES >= 32) {
    const unsigned u = __builtin_bit_cast(unsigned, v);
    const u32x2 r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    const unsigned even = r.x, odd = r.y;
    v = op(__builtin_bit_cast(float, even), __builtin_bit_cast(float, odd));
  }
  if (LANES >= 64) {
    const unsigned u = __builtin_bit_cast(unsigned, v);
    const u32x2 r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    const unsigned lo = r.x, hi = r.y;
    v = op(__builtin_bit_cast(float, lo), __builtin_bit_cast(float, hi));
  }
  return v;
}

// Reduction of `v` over all TPR lanes of a row.  `red` holds one float per
// wave of the workgroup; with one wave per row it is never touched.
template <class Op>
__device__ __forceinline__ float row_reduce(float v, Op op, float* red, int row_in_block,
                                            int wave_in_row, int lane) {
  v = wave_allreduce<RED_LANES>(v, op);
#if NW > 1
  float* slot = red + row_in_block * NW;
  if (lane == 0) slot[wave_in_row] = v;
  __syncthreads();
  float r = slot[0];
#pragma unroll
  for (int i = 1; i < NW; ++i) r = op(r, slot[i]);
  v = r;
#endif
  return v;
}

// ---------------------------------------------------------------------------
// memory helpers
// ---------------------------------------------------------------------------
__device__ __forceinline__ vec_t load_vec(const elem_t* p, bool once) {
#if DECA_HINT
  if (once) return __builtin_nontemporal_load(reinterpret_cast<const vec_t*>(p));
#endif
  return *reinterpret_cast<const vec_t*>(p);
}

__device__ __forceinline__ void store_vec(elem_t* p, vec_t v) {
#if DECA_HINT
  __builtin_nontemporal_store(v, reinterpret_cast<vec_t*>(p));
#else
  *reinterpret_cast<vec_t*>(p) = v;
#endif
}

__device__ __forceinline__ float fast_exp2(float v) { return __builtin_amdgcn_exp2f(v); }

// ---------------------------------------------------------------------------
// kernel
// ---------------------------------------------------------------------------
extern "C" __global__ void __launch_bounds__(NT)
deca_main(const elem_t* __restrict__ x,
#if DECA_OP == 1
          const elem_t* __restrict__ w,
#endif
          elem_t* __restrict__ y) {
#if NW > 1
  __shared__ float red_lds[2 * RPB * NW];
  float* red0 = red_lds;
  float* red1 = red_lds + RPB * NW;
#else
  float* red0 = nullptr;
  float* red1 = nullptr;
#endif
  const int tid = threadIdx.x;
  const int t = tid % TPR;
  const int rb = tid / TPR;
  const int lane = tid % 64;
  const int wr = t / 64;
  const size_t row_base = (static_cast<size_t>(blockIdx.x) * RPB + rb) * DECA_N;
  const elem_t* xr = x + row_base;
  elem_t* yr = y + row_base;

  auto col = [&](int c) { return (c * TPR + t) * VEC; };
  // Chunks >= C_FULL are out of the row for the upper lanes.
  auto in_row = [&](int c) { return c < C_FULL || col(c) < DECA_N; };

#if DECA_MODE == 0
  // ------------------------------ reg mode ------------------------------
  vec_t xh[NCHUNK];
#pragma unroll
  for (int c = 0; c < NCHUNK; ++c) {
    if (in_row(c)) xh[c] = load_vec(xr + col(c), true);
  }

#if DECA_OP == 0
  float m = NEG_INF;
#pragma unroll
  for (int c = 0; c < NCHUNK; ++c) {
    const bool ok = in_row(c);
#pragma unroll
    for (int i = 0; i < VEC; ++i) m = fmaxf(m, ok ? static_cast<float>(xh[c][i]) : NEG_INF);
  }
  const float m2 = row_reduce(m, MaxOp(), red0, rb, wr, lane) * LOG2E;
#if DECA_LEAN
  // (see below: the fp32 conversions of the max pass are not kept for the sum)
#pragma unroll
  for (int c = 0; c < NCHUNK; ++c) asm volatile("" : "+v"(xh[c]));
#endif
  float s = 0.0f;
#pragma unroll
  for (int c = 0; c < NCHUNK; ++c) {
    const bool ok = in_row(c);
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      const float v = ok ? static_cast<float>(xh[c][i]) : NEG_INF;
      s += fast_exp2(v * LOG2E - m2);
    }
  }
  const float inv = __builtin_amdgcn_rcpf(row_reduce(s, AddOp(), red1, rb, wr, lane));
#if DECA_LEAN
  // The optimiser would keep the exponentials of the sum alive for the stores
  // (2 VGPRs per element on top of the packed row).  Reading the row through an
  // opaque copy makes it compute them again from the same bits instead.
#pragma unroll
  for (int c = 0; c < NCHUNK; ++c) asm volatile("" : "+v"(xh[c]));
#endif
#pragma unroll
  for (int c = 0; c < NCHUNK; ++c) {
    if (in_row(c)) {
      vec_t o;
#pragma unroll
      for (int i = 0; i < VEC; ++i)
        o[i] = static_cast<elem_t>(fast_exp2(static_cast<float>(xh[c][i]) * LOG2E - m2) * inv);
      store_vec(yr + col(c), o);
    }
  }
#else
  float ss = 0.0f;
#pragma unroll
  for (int c = 0; c < NCHUNK; ++c) {
    const bool ok = in_row(c);
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      const float v = ok ? static_cast<float>(xh[c][i]) : 0.0f;
      ss += v * v;
    }
  }
  ss = row_reduce(ss, AddOp(), red0, rb, wr, lane);
  const float r = __builtin_amdgcn_rsqf(ss * (1.0f / DECA_N) + static_cast<float>(DECA_EPS));
#if DECA_LEAN
  // as above: the fp32 conversions of the row are made again, not kept
#pragma unroll
  for (int c = 0; c < NCHUNK; ++c) asm volatile("" : "+v"(xh[c]));
#endif
#pragma unroll
  for (int c = 0; c < NCHUNK; ++c) {
    if (in_row(c)) {
      const vec_t wv = *reinterpret_cast<const vec_t*>(w + col(c));
      vec_t o;
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        const float normed = static_cast<float>(static_cast<elem_t>(static_cast<float>(xh[c][i]) * r));
        o[i] = static_cast<elem_t>(normed * static_cast<float>(wv[i]));
      }
      store_vec(yr + col(c), o);
    }
  }
#endif

#else
  // ----------------------------- twopass mode -----------------------------
  constexpr int U = DECA_UNROLL;
  constexpr int N_LOOP = C_FULL / U;  // iterations whose U chunks are all in the row

#if DECA_OP == 0
  float run_m = NEG_INF;  // running max, already scaled by log2e
  float run_s = 0.0f;
  auto online = [&](const vec_t* v, const bool* ok, int n) {
    float mx = run_m;
#pragma unroll
    for (int u = 0; u < n; ++u)
#pragma unroll
      for (int i = 0; i < VEC; ++i)
        mx = fmaxf(mx, ok[u] ? static_cast<float>(v[u][i]) * LOG2E : NEG_INF);
    float acc = 0.0f;
#pragma unroll
    for (int u = 0; u < n; ++u)
#pragma unroll
      for (int i = 0; i < VEC; ++i)
        acc += fast_exp2((ok[u] ? static_cast<float>(v[u][i]) * LOG2E : NEG_INF) - mx);
    run_s = run_s * fast_exp2(run_m - mx) + acc;
    run_m = mx;
  };
#else
  float run_ss = 0.0f;
  auto online = [&](const vec_t* v, const bool* ok, int n) {
    float acc = 0.0f;
#pragma unroll
    for (int u = 0; u < n; ++u)
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        const float f = ok[u] ? static_cast<float>(v[u][i]) : 0.0f;
        acc += f * f;
      }
    run_ss += acc;
  };
#endif

  // pass 1: the row is read again soon, so it is loaded with the default policy
  for (int g = 0; g < N_LOOP; ++g) {
    vec_t v[U];
    bool ok[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      v[u] = load_vec(xr + col(g * U + u), false);
      ok[u] = true;
    }
    online(v, ok, U);
  }
#pragma unroll
  for (int c = N_LOOP * U; c < NCHUNK; ++c) {
    vec_t v[1];
    bool ok[1];
    ok[0] = in_row(c);
    if (ok[0]) v[0] = load_vec(xr + col(c), false);
    online(v, ok, 1);
  }

#if DECA_OP == 0
  const float m2 = row_reduce(run_m, MaxOp(), red0, rb, wr, lane);
  const float tot = row_reduce(run_s * fast_exp2(run_m - m2), AddOp(), red1, rb, wr, lane);
  const float inv = __builtin_amdgcn_rcpf(tot);
  auto emit = [&](int c, vec_t v) {
    vec_t o;
#pragma unroll
    for (int i = 0; i < VEC; ++i)
      o[i] = static_cast<elem_t>(fast_exp2(static_cast<float>(v[i]) * LOG2E - m2) * inv);
    store_vec(yr + col(c), o);
  };
#else
  const float tot = row_reduce(run_ss, AddOp(), red0, rb, wr, lane);
  const float r = __builtin_amdgcn_rsqf(tot * (1.0f / DECA_N) + static_cast<float>(DECA_EPS));
  auto emit = [&](int c, vec_t v) {
    const vec_t wv = *reinterpret_cast<const vec_t*>(w + col(c));
    vec_t o;
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      const float normed = static_cast<float>(static_cast<elem_t>(static_cast<float>(v[i]) * r));
      o[i] = static_cast<elem_t>(normed * static_cast<float>(wv[i]));
    }
    store_vec(yr + col(c), o);
  };
#endif

  // pass 2: last use of the row
  for (int g = 0; g < N_LOOP; ++g) {
    vec_t v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) v[u] = load_vec(xr + col(g * U + u), true);
#pragma unroll
    for (int u = 0; u < U; ++u) emit(g * U + u, v[u]);
  }
#pragma unroll
  for (int c = N_LOOP * U; c < NCHUNK; ++c) {
    if (in_row(c)) emit(c, load_vec(xr + col(c), true));
  }
#endif
}
