// Decode-form 4-bit matmuls for 1..16 rows an item: the routed-expert GEMV (tf_experts_run) and the dense lane
// matmul (tf_qmm), plus tf_group_sums.  HBM-bound: one pass over the packed weights.
//
// Mapping.  A lane owns one output column and walks K; the 64 lanes of a wave read 1 KB of codes with one
// 16-byte load each (a chunk: 32 inputs x 64 columns).  The activations of the item's rows are wave-uniform, so
// they come through scalar loads and feed v_dot2c_f32_bf16 straight from SGPRs: no cross-lane reduction is
// needed and the vector memory pipe carries weights only.  The waves of a workgroup split the groups of K
// (a function of the shape alone) and their fp32 partials are added through LDS in wave order, so a row's bits
// never depend on the other rows of the call.
//
// Arithmetic per group, as the reference's decode form (experts.cu:94-106, qmm.cu:66-76):
//   acc = fma(xs, b, fma(P, s, acc)),   P = sum x * q,   xs = sum x
// with q exact: a nibble OR-ed into the bf16 pattern of 128 is 128 + q, so the dot product gives P + 128 xs and
// P = fma(-128, xs, that).

#include "tf_common.h"

namespace tf {
namespace {

typedef const __attribute__((address_space(4))) uint32_t* const_u32_ptr;   // constant address space: scalar loads

__device__ __forceinline__ const_u32_ptr as_const(const void* p) {
  return (const_u32_ptr)(reinterpret_cast<uintptr_t>(p));
}

__device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float c) {
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, a), __builtin_bit_cast(bf16x2_t, b), c, false);
}

__device__ __forceinline__ uint4 ldg16(const uint32_t* p) { return *reinterpret_cast<const uint4*>(p); }

// fp32 sums of each group of GS inputs of `rows` rows, for groups [0, KG), into xs[r * KG + g].
// LPG lanes share a group (8 inputs each, in order), then a fixed xor tree over them.
template <int GS>
__device__ __forceinline__ void group_sums_block(const uint16_t* const* xrow, int rows, int KG, float* xs, int tid,
                                                 int threads) {
  constexpr int LPG = GS / 8;
  const int part = tid % LPG;
  for (int r = 0; r < rows; ++r) {
    for (int g = tid / LPG; g < KG; g += threads / LPG) {
      const uint4 v = *reinterpret_cast<const uint4*>(xrow[r] + (size_t)g * GS + part * 8);
      float s = bf16_lo(v.x);
      s += bf16_hi(v.x);
      s += bf16_lo(v.y);
      s += bf16_hi(v.y);
      s += bf16_lo(v.z);
      s += bf16_hi(v.z);
      s += bf16_lo(v.w);
      s += bf16_hi(v.w);
#pragma unroll
      for (int m = 1; m < LPG; m <<= 1) s += __shfl_xor(s, m);
      if (part == 0) xs[r * KG + g] = s;
    }
  }
}

// (x & mask) | magic in one VALU op; the mask rides in an SGPR and the magic in a VGPR (one constant-bus read)
__device__ __forceinline__ uint32_t and_or(uint32_t x, uint32_t mask, uint32_t magic) {
  uint32_t r;
  asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(x), "s"(mask), "v"(magic));
  return r;
}

// A group's weights of NM matrices in registers: GS/32 16-byte chunks and the (scale | bias << 16) word a matrix.
template <int GS, int NM>
struct Stage {
  uint4 w[NM][GS / 32];
  float s[NM], b[NM];
};

template <int GS, int NM, class WQ, class SB>
__device__ __forceinline__ void load_stage(Stage<GS, NM>& st, const WQ& wq, const SB& sb, int g) {
#pragma unroll
  for (int m = 0; m < NM; ++m) {
#pragma unroll
    for (int i = 0; i < GS / 32; ++i) st.w[m][i] = wq(g, m, i);
    sb(g, m, st.s[m], st.b[m]);
  }
}

// acc += one group: P = sum x * (128 + q) by v_dot2c (x from SGPRs), then the scale and bias.
template <int GS, int NM, int RB>
__device__ __forceinline__ void compute_stage(float (&acc)[NM][RB], const Stage<GS, NM>& st,
                                              const const_u32_ptr (&xr)[RB], const float* xs, int KG, int g) {
  constexpr int CH = GS / 32;
  const uint32_t magic = BF16_128;
#ifdef TF_X_NOCOMPUTE
#pragma unroll
  for (int m = 0; m < NM; ++m)
#pragma unroll
    for (int i = 0; i < CH; ++i)
      acc[m][0] += __uint_as_float((st.w[m][i].x ^ st.w[m][i].y ^ st.w[m][i].z ^ st.w[m][i].w) & 0x3fffffffu) + st.s[m] + st.b[m];
  return;
#endif
  float p[NM][RB];
#pragma unroll
  for (int m = 0; m < NM; ++m)
#pragma unroll
    for (int r = 0; r < RB; ++r) p[m][r] = 0.f;
#pragma unroll
  for (int i = 0; i < CH; ++i) {
    uint32_t xv[RB][16];
#pragma unroll
    for (int r = 0; r < RB; ++r)
#pragma unroll
#ifdef TF_X_NOX
      for (int j = 0; j < 16; ++j) xv[r][j] = 0x3f803f80u + (uint32_t)KG;
#else
      for (int j = 0; j < 16; ++j) xv[r][j] = xr[r][(g * CH + i) * 16 + j];
#endif
#pragma unroll
    for (int m = 0; m < NM; ++m) {
      const uint32_t w4[4] = {st.w[m][i].x, st.w[m][i].y, st.w[m][i].z, st.w[m][i].w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const uint32_t b2 = and_or(q ? w4[j] >> (4 * q) : w4[j], NIB_MASK, magic);
#pragma unroll
          for (int r = 0; r < RB; ++r) p[m][r] = dot2(b2, xv[r][4 * j + q], p[m][r]);
        }
      }
    }
  }
#pragma unroll
  for (int r = 0; r < RB; ++r) {
    const float xsum = xs[r * KG + g];
#pragma unroll
    for (int m = 0; m < NM; ++m) {
      const float pq = fmaf(-128.f, xsum, p[m][r]);
      acc[m][r] = fmaf(xsum, st.b[m], fmaf(pq, st.s[m], acc[m][r]));
    }
  }
}

#ifndef TF_X_DEPTH
#define TF_X_DEPTH 3
#endif
constexpr int DEPTH = TF_X_DEPTH;        // groups a wave keeps in flight

// One wave's share of a GEMV: groups [g0, g1) of NM matrices against RB rows, DEPTH groups in flight.
//   wq(g, m, i)  -> the lane's 16 bytes of chunk i of group g of matrix m
//   sb(g, m, s, b) -> the lane's column's scale and bias of that group
//   xr[r]        -> row r's inputs as dwords (wave-uniform, constant address space)
//   xs[r * KG + g] -> group sums (LDS)
// `st` holds groups g0 .. g0 + DEPTH - 1 on entry when `loaded` (the caller issued them before its prologue).
template <int GS, int NM, int RB, class WQ, class SB>
__device__ __forceinline__ void gemv_slice(float (&acc)[NM][RB], Stage<GS, NM> (&st)[DEPTH], bool loaded, const WQ& wq,
                                           const SB& sb, const const_u32_ptr (&xr)[RB], const float* xs, int KG,
                                           int g0, int g1) {
  if (!loaded) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d)
      if (g0 + d < g1) load_stage<GS, NM>(st[d], wq, sb, g0 + d);
  }
  for (int gb = g0; gb < g1; gb += DEPTH) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      const int g = gb + d;
      if (g < g1) {
        compute_stage<GS, NM, RB>(acc, st[d], xr, xs, KG, g);
        if (g + DEPTH < g1) load_stage<GS, NM>(st[d], wq, sb, g + DEPTH);
      }
    }
  }
}

// ---- routed experts -----------------------------------------------------------------------------------------------

// One pass of an item: RB of its rows (first + r0 ..) against the workgroup's 64 columns.
template <int GS, int NM, int EPI, int WAVES, int RB, class WQ, class SB>
__device__ __forceinline__ void expert_pass(const uint16_t* __restrict__ X, int64_t x_stride, int slots, const WQ& wq,
                                            const SB& sb, int KG, int NB, int cb2, const int* __restrict__ members,
                                            int at0, void* __restrict__ out, int N, float limit, float* xs, float* part,
                                            int g0, int g1, Stage<GS, NM> (&st)[DEPTH], bool loaded) {
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  int pr[RB];
  const uint16_t* xrow[RB];
  const_u32_ptr xr[RB];
#pragma unroll
  for (int r = 0; r < RB; ++r) {
    pr[r] = members[at0 + r];
    const int row = slots ? pr[r] / slots : pr[r];
    xrow[r] = X + (size_t)row * x_stride;
    xr[r] = as_const(xrow[r]);
  }
  __syncthreads();                                  // the previous pass is done with xs and part
#ifndef TF_X_NOXS
  group_sums_block<GS>(xrow, RB, KG, xs, tid, WAVES * 64);
  __syncthreads();
#endif
  float acc[NM][RB];
#pragma unroll
  for (int m = 0; m < NM; ++m)
#pragma unroll
    for (int r = 0; r < RB; ++r) acc[m][r] = 0.f;
  gemv_slice<GS, NM, RB>(acc, st, loaded, wq, sb, xr, xs, KG, g0, g1);
#pragma unroll
  for (int m = 0; m < NM; ++m)
#pragma unroll
    for (int r = 0; r < RB; ++r) part[((wave * NM + m) * RB + r) * 64 + lane] = acc[m][r];
  __syncthreads();
  // thread (r, column): the waves' partials in wave order, then the epilogue
  for (int o = tid; o < RB * 64; o += WAVES * 64) {
    const int r = o >> 6, l = o & 63;
    const int onb = 2 * cb2 + (l >> 5);
    if (onb >= NB) continue;
    float v[NM];
#pragma unroll
    for (int m = 0; m < NM; ++m) {
      float s = part[(m * RB + r) * 64 + l];
      for (int w = 1; w < WAVES; ++w) s += part[((w * NM + m) * RB + r) * 64 + l];
      v[m] = s;
    }
    int prow = pr[0];
#pragma unroll
    for (int q = 1; q < RB; ++q) prow = r == q ? pr[q] : prow;
    const size_t at = (size_t)prow * N + onb * 32 + (l & 31);
    if constexpr (EPI == 0) {
      reinterpret_cast<float*>(out)[at] = v[0];
    } else if constexpr (EPI == 1) {
      reinterpret_cast<uint16_t*>(out)[at] = (uint16_t)f32_bf16_bits(relu2(v[0]));
    } else {
      reinterpret_cast<uint16_t*>(out)[at] = (uint16_t)f32_bf16_bits(swiglu(v[0], v[NM - 1], limit));
    }
  }
}

// A workgroup takes (item, pair of 32-column blocks): lanes 0-31 the even block, lanes 32-63 the odd one.
// Pair p reads X row p / slots when slots > 0, else row p (experts.cu:129).  The item's rows go through in passes
// of 4, 2 or 1; a row's arithmetic is the same in each, so its bits do not depend on the pass it lands in.
template <int GS, int NM, int EPI, int WAVES>
__global__ void __launch_bounds__(WAVES * 64)
    expert_kernel(const uint16_t* __restrict__ X, int64_t x_stride, int slots, const uint32_t* __restrict__ W, int KG,
                  int NB, const int* __restrict__ items, const int* __restrict__ counts,
                  const int* __restrict__ members, void* __restrict__ out, int N, float limit) {
  constexpr int BW = block_words(GS);
  extern __shared__ float lds[];            // xs [4][KG], then partials [WAVES][NM][4][64]
  const int NB2 = (NB + 1) >> 1;
  const int it = blockIdx.x / NB2, cb2 = blockIdx.x - it * NB2;
#ifdef TF_X_NOITEM
  if (it >= 40) return;
  const int e = it * 3 + 1, first = it, cnt = 1;
#else
  if (it >= counts[0]) return;
  const int e = items[3 * it], first = items[3 * it + 1], cnt = items[3 * it + 2];
#endif
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int nb = 2 * cb2 + (lane >> 5), c = lane & 31;
  const bool col_ok = nb < NB;
  const uint32_t* wbase =
      W + (((size_t)e * NB + (col_ok ? nb : NB - 1)) * KG) * (size_t)(NM * BW) + c * 4;
  const uint32_t* sbase = wbase - c * 4 + 32 * GS / 8 + c;
  auto wq = [&](int g, int m, int i) { return ldg16(wbase + ((size_t)g * NM + m) * BW + i * 128); };
  auto sb = [&](int g, int m, float& s, float& b) {
    const uint32_t v = sbase[((size_t)g * NM + m) * BW];
    s = bf16_lo(v);
    b = bf16_hi(v);
  };
  const int g0 = (int)((long long)wave * KG / WAVES), g1 = (int)((long long)(wave + 1) * KG / WAVES);
  float* xs = lds;
  float* part = lds + 4 * KG;
  // the slice's first groups are on their way before anything else is read
  Stage<GS, NM> st[DEPTH];
#pragma unroll
  for (int d = 0; d < DEPTH; ++d)
    if (g0 + d < g1) load_stage<GS, NM>(st[d], wq, sb, g0 + d);
  bool loaded = true;
  int r0 = 0;
#define TF_PASS(RB_)                                                                                                 \
  expert_pass<GS, NM, EPI, WAVES, RB_>(X, x_stride, slots, wq, sb, KG, NB, cb2, members, first + r0, out, N, limit, xs, \
                                       part, g0, g1, st, loaded);                                                    \
  loaded = g1 - g0 <= DEPTH   /* a slice that fits the stages stays in registers for the next pass */
  for (; r0 + 4 <= cnt; r0 += 4) {
    TF_PASS(4);
  }
  if (r0 + 2 <= cnt) {
    TF_PASS(2);
    r0 += 2;
  }
  if (r0 < cnt) {
    TF_PASS(1);
  }
#undef TF_PASS
}

// ---- dense lane matmul ---------------------------------------------------------------------------------------------

// One pass of a row tile: RB rows r0 .. r0 + RB - 1 against the workgroup's 64 columns and K slice.
template <int GS, int WAVES, int RB, class WQ, class SB>
__device__ __forceinline__ void qmm_pass(const uint16_t* __restrict__ X, int64_t ldx, const float* __restrict__ XS,
                                         const WQ& wq, const SB& sb, int r0, int tile, int slice, int gs0, int per,
                                         int g0, int g1, void* __restrict__ out, float* __restrict__ part_out, int M,
                                         int N, int KG, int SK, int f32, float* xs, float* part,
                                         Stage<GS, 1> (&st)[DEPTH], bool loaded) {
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const_u32_ptr xr[RB];
#pragma unroll
  for (int r = 0; r < RB; ++r) xr[r] = as_const(X + (size_t)(r0 + r) * ldx);
  __syncthreads();
  for (int o = tid; o < RB * per; o += WAVES * 64) {
    const int r = o / per, g = o - r * per;
    xs[r * per + g] = XS[(size_t)(r0 + r) * KG + gs0 + g];
  }
  __syncthreads();
  float acc[1][RB];
#pragma unroll
  for (int r = 0; r < RB; ++r) acc[0][r] = 0.f;
  // gemv_slice indexes xs by absolute group: shift the base so that xs[r * per + (g - gs0)] is read
  gemv_slice<GS, 1, RB>(acc, st, loaded, wq, sb, xr, xs - gs0, per, g0, g1);
#pragma unroll
  for (int r = 0; r < RB; ++r) part[(wave * RB + r) * 64 + lane] = acc[0][r];
  __syncthreads();
  for (int o = tid; o < RB * 64; o += WAVES * 64) {
    const int r = o >> 6, l = o & 63, cc = tile * 64 + l;
    if (cc >= N) continue;
    float s = part[r * 64 + l];
    for (int w = 1; w < WAVES; ++w) s += part[(w * RB + r) * 64 + l];
    const size_t at = (size_t)(r0 + r) * N + cc;
    if (SK > 1) part_out[(size_t)slice * M * N + at] = s;
    else if (f32) reinterpret_cast<float*>(out)[at] = s;
    else reinterpret_cast<uint16_t*>(out)[at] = (uint16_t)f32_bf16_bits(s);
  }
}

// grid (column tiles of 64 x row tiles of BM, 1, SK).  Slice z takes groups [z * per, (z + 1) * per), its waves
// split them again; SK > 1 leaves the slice's fp32 sums in part[z].  Rows go through in passes of 4, 2 or 1.
template <int GS, int WAVES>
__global__ void __launch_bounds__(WAVES * 64)
    qmm_kernel(const uint16_t* __restrict__ X, int64_t ldx, const float* __restrict__ XS,
               const uint32_t* __restrict__ W, const uint16_t* __restrict__ S, const uint16_t* __restrict__ B,
               int64_t sb_stride, void* __restrict__ out, float* __restrict__ part_out, int M, int N, int KG, int SK,
               int BM, int f32) {
  extern __shared__ float lds[];            // xs [4][per], then partials [WAVES][4][64]
  const int tiles = (N + 63) >> 6;
  const int tile = blockIdx.x % tiles, rt = blockIdx.x / tiles, slice = blockIdx.z;
  const int per = KG / SK, gs0 = slice * per;
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  constexpr int CH = GS / 32;
  const uint32_t* wbase = W + ((size_t)tile * KG) * (size_t)(CH * 256) + lane * 4;
  const int col = tile * 64 + lane;
  auto wq = [&](int g, int m, int i) { return ldg16(wbase + ((size_t)g * CH + i) * 256); };
  auto sb = [&](int g, int m, float& s, float& b) {
    s = bf16_f32(S[(size_t)g * sb_stride + col]);
    b = bf16_f32(B[(size_t)g * sb_stride + col]);
  };
  const int g0 = gs0 + (int)((long long)wave * per / WAVES), g1 = gs0 + (int)((long long)(wave + 1) * per / WAVES);
  float* xs = lds;
  float* part = lds + 4 * per;
  const int m_end = min(M, (rt + 1) * BM);
  int r0 = rt * BM;
  Stage<GS, 1> st[DEPTH];
#pragma unroll
  for (int d = 0; d < DEPTH; ++d)
    if (g0 + d < g1) load_stage<GS, 1>(st[d], wq, sb, g0 + d);
  bool loaded = true;
#define TF_QMM_PASS(RB_)                                                                                             \
  qmm_pass<GS, WAVES, RB_>(X, ldx, XS, wq, sb, r0, tile, slice, gs0, per, g0, g1, out, part_out, M, N, KG, SK, f32, xs, \
                           part, st, loaded);                                                                        \
  loaded = g1 - g0 <= DEPTH
  for (; r0 + 4 <= m_end; r0 += 4) {
    TF_QMM_PASS(4);
  }
  if (r0 + 2 <= m_end) {
    TF_QMM_PASS(2);
    r0 += 2;
  }
  if (r0 < m_end) {
    TF_QMM_PASS(1);
  }
#undef TF_QMM_PASS
}

// the K slices' partial sums added in slice order, then rounded once (qmm.cu:222-230)
__global__ void qmm_reduce_kernel(const float* __restrict__ part, void* __restrict__ out, long long total, int SK,
                                  int f32) {
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  float acc = part[i];
  for (int s = 1; s < SK; ++s) acc = acc + part[s * total + i];
  if (f32) reinterpret_cast<float*>(out)[i] = acc;
  else reinterpret_cast<uint16_t*>(out)[i] = (uint16_t)f32_bf16_bits(acc);
}

template <int GS>
__global__ void __launch_bounds__(256)
    group_sums_kernel(const uint16_t* __restrict__ X, int64_t ldx, int M, int KG, float* __restrict__ XS) {
  const int r = blockIdx.x;
  const uint16_t* xrow[1] = {X + (size_t)r * ldx};
  group_sums_block<GS>(xrow, 1, KG, XS + (size_t)r * KG, threadIdx.x, 256);
}

#ifndef TF_X_WAVES
#define TF_X_WAVES 16
#endif
constexpr int EXPERT_WAVES = TF_X_WAVES;
constexpr int EXPERT_RB = 4;
constexpr int QMM_WAVES = 4;
constexpr int QMM_RB = 4;

template <int GS, int NM, int EPI>
int launch_experts(const uint16_t* x, int64_t x_stride, int slots, const uint32_t* w, int kg, int nb, const int* items,
                   const int* counts, const int* members, void* out, int n, float limit, int64_t max_units,
                   hipStream_t stream) {
  const int nb2 = (nb + 1) / 2;
  const int64_t max_items = (max_units + nb - 1) / nb;
  const int64_t grid = max_items * nb2;
  if (grid < 1) return 0;
  TF_REQUIRE(grid <= 0x7FFFFFFF, "experts: %lld workgroups exceed the grid limit", (long long)grid);
  const size_t smem = sizeof(float) * ((size_t)EXPERT_RB * kg + (size_t)EXPERT_WAVES * NM * EXPERT_RB * 64);
  TF_REQUIRE(smem <= 64 * 1024, "experts: K/gs = %d groups need %zu bytes of LDS (limit 65536)", kg, smem);
  expert_kernel<GS, NM, EPI, EXPERT_WAVES><<<dim3((unsigned)grid), dim3(EXPERT_WAVES * 64), smem, stream>>>(
      x, x_stride, slots, w, kg, nb, items, counts, members, out, n, limit);
  TF_LAUNCH_OK("tf_experts_run");
  return 0;
}

}  // namespace
}  // namespace tf

using namespace tf;

extern "C" int tf_experts_run(int gs, int epi, const uint16_t* x, int64_t x_stride, int slots, const uint32_t* w,
                              int kg, int nb, const int32_t* items, const int32_t* counts, const int32_t* members,
                              void* out, int n, float limit, int64_t max_units, tf_stream_t stream) {
  clear_error();
  TF_REQUIRE(gs == 32 || gs == 64, "experts: groups of 32 or 64 inputs, not %d", gs);
  TF_REQUIRE(x && w && items && counts && members && out, "experts: null pointer argument");
  TF_REQUIRE(kg >= 1 && nb >= 1 && n == nb * 32, "experts: n (%d) must be the column blocks (%d) times 32", n, nb);
  TF_REQUIRE(aligned16(x) && x_stride % 8 == 0, "x: rows of K = groups * group size inputs, 16-byte aligned");
  TF_REQUIRE(aligned16(w), "w must be 16-byte aligned");
  TF_REQUIRE(slots >= 0 && max_units >= 0, "experts: negative slots or max_units");
  hipStream_t s = as_stream(stream);
#define TF_RUN(GS_, NM_, EPI_) \
  if (gs == GS_ && epi == EPI_) \
    return launch_experts<GS_, NM_, EPI_>(x, x_stride, slots, w, kg, nb, items, counts, members, out, n, limit, max_units, s);
  TF_RUN(32, 1, 0) TF_RUN(32, 1, 1) TF_RUN(32, 2, 2) TF_RUN(64, 1, 0) TF_RUN(64, 1, 1) TF_RUN(64, 2, 2)
#undef TF_RUN
  set_error("experts: no kernel for group %d and epilogue %d", gs, epi);
  return 1;
}

extern "C" int tf_group_sums(const uint16_t* x, int64_t ldx, int m, int k, int gs, float* xs, tf_stream_t stream) {
  clear_error();
  TF_REQUIRE(gs == 32 || gs == 64, "group_sums: groups of 32 or 64 inputs, not %d", gs);
  TF_REQUIRE(x && xs && m >= 1 && k >= gs && k % gs == 0, "group_sums: x must be (M, K), K a multiple of the group");
  TF_REQUIRE(aligned16(x) && (m == 1 || ldx % 8 == 0), "x rows must start on 16-byte boundaries");
  if (gs == 64) group_sums_kernel<64><<<m, 256, 0, as_stream(stream)>>>(x, ldx, m, k / gs, xs);
  else group_sums_kernel<32><<<m, 256, 0, as_stream(stream)>>>(x, ldx, m, k / gs, xs);
  TF_LAUNCH_OK("tf_group_sums");
  return 0;
}

extern "C" int tf_qmm(const uint16_t* x, int64_t ldx, const float* xs, const uint32_t* weight, const uint16_t* scales,
                      const uint16_t* biases, int64_t sb_stride, void* out, float* part, int m, int n, int k, int sk,
                      int gs, int bm, int f32, int reduce, tf_stream_t stream) {
  clear_error();
  TF_REQUIRE(gs == 32 || gs == 64, "groups of 32 or 64");
  TF_REQUIRE(bm == 16 || bm == 32 || bm == 64, "row tile 16, 32 or 64");
  TF_REQUIRE(x && xs && weight && scales && biases && out && m >= 1 && n >= 1, "qmm: null pointer or empty shape");
  TF_REQUIRE(aligned16(x) && (m == 1 || ldx % 8 == 0), "x rows must start on 16-byte boundaries");
  TF_REQUIRE(ldx >= k || m == 1, "x: (M, K) bf16 with contiguous rows");
  const int kg = k / gs, npad = (n + 127) / 128 * 128;
  TF_REQUIRE(k % gs == 0 && sk >= 1 && kg % sk == 0, "K splits into whole groups a slice");
  TF_REQUIRE(sb_stride >= npad, "scales and biases: (K / gs, n padded to 128) bf16, rows may be strided");
  TF_REQUIRE(aligned16(weight), "packed weight must be 16-byte aligned");
  TF_REQUIRE(sk == 1 || part, "part: at least (SK, M, n) fp32 is needed when K is split");
  hipStream_t s = as_stream(stream);
  const int tiles = (n + 63) / 64, rts = (m + bm - 1) / bm, per = kg / sk;
  const size_t smem = sizeof(float) * ((size_t)QMM_RB * per + (size_t)QMM_WAVES * QMM_RB * 64);
  TF_REQUIRE(smem <= 64 * 1024, "qmm: %d groups a slice need %zu bytes of LDS (limit 65536)", per, smem);
  TF_REQUIRE((int64_t)tiles * rts <= 0x7FFFFFFF && sk <= 65535, "qmm: grid too large");
  const dim3 grid((unsigned)(tiles * rts), 1, (unsigned)sk);
  if (gs == 64)
    qmm_kernel<64, QMM_WAVES><<<grid, QMM_WAVES * 64, smem, s>>>(x, ldx, xs, weight, scales, biases, sb_stride,
                                                                       out, part, m, n, kg, sk, bm, f32);
  else
    qmm_kernel<32, QMM_WAVES><<<grid, QMM_WAVES * 64, smem, s>>>(x, ldx, xs, weight, scales, biases, sb_stride,
                                                                       out, part, m, n, kg, sk, bm, f32);
  TF_LAUNCH_OK("tf_qmm");
  if (sk > 1 && reduce) {
    const long long total = (long long)m * n;
    qmm_reduce_kernel<<<(unsigned)((total + 255) / 256), 256, 0, s>>>(part, out, total, sk, f32);
    TF_LAUNCH_OK("tf_qmm reduce");
  }
  return 0;
}
