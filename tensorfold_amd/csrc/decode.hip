// Decode-form 4-bit matmuls for 1..16 rows an item: the routed-expert GEMV (tf_experts_run) and the dense lane
// matmul (tf_qmm), plus tf_group_sums.  HBM-bound: one pass over the packed weights.
//
// Mapping.  A lane owns one output column and walks K; the 64 lanes of a wave read 1 KB of codes with one
// 16-byte load each (a chunk: 32 inputs x 64 columns).  The activations of the item's rows are the same for every
// lane: each lane loads dword (lane % 16) of the chunk (one coalesced 64-byte read, fetched with the weights,
// DEPTH groups ahead) and v_dot2c_f32_bf16's DPP form broadcasts dword j across each row of 16 lanes inside the
// multiply itself (row_newbcast:j), so there is no cross-lane reduction, no scalar-cache traffic and no LDS
// traffic in the inner loop.
//
// K is cut into SLICES fixed slices (a function of the shape alone).  A workgroup's waves each walk a run of
// consecutive slices, park each slice's fp32 sum in LDS, and the sums are added in slice order; how many waves
// share the slices (16, 8 or 4, picked from the launch size) therefore never changes a bit, and neither do the
// other rows of the call.
//
// Arithmetic per group, as the reference's decode form (experts.cu:94-106, qmm.cu:66-76):
//   acc = fma(xs, b, fma(P, s, acc)),   P = sum x * q,   xs = sum x
// with q exact: a nibble OR-ed into the bf16 pattern of 128 is 128 + q, so the dot product gives P + 128 xs and
// P = fma(-128, xs, that).

#include <cstdlib>

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

// weights are read once: nontemporal loads keep them from displacing the activations in the caches
__device__ __forceinline__ uint4 ldg16(const uint32_t* p) {
#ifdef TF_X_TEMPORAL
  return *reinterpret_cast<const uint4*>(p);
#else
  const u32x4_t v = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(p));
  return make_uint4(v.x, v.y, v.z, v.w);
#endif
}

// (x & mask) | magic in one VALU op; the mask rides in an SGPR and the magic in a VGPR (one constant-bus read)
__device__ __forceinline__ uint32_t and_or(uint32_t x, uint32_t mask, uint32_t magic) {
  uint32_t r;
  asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(x), "s"(mask), "v"(magic));
  return r;
}

constexpr int SLICES = 16;      // K slices of the expert GEMV
constexpr int DEPTH = 3;        // groups of weights a wave keeps in flight
constexpr int RBMAX = 2;        // rows a pass

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

// dot2c with its first operand taken from lane J of the reader's row of 16 lanes
template <int J>
__device__ __forceinline__ float dot2_bcast(float acc, uint32_t x, uint32_t q) {
  asm("v_dot2c_f32_bf16_dpp %0, %1, %2 row_newbcast:%3 row_mask:0xf bank_mask:0xf" : "+v"(acc) : "v"(x), "v"(q), "n"(J));
  return acc;
}

// A group in registers: the weights of NM matrices (GS/32 16-byte chunks, scale and bias) and, of each of RB rows,
// the lane's dword of each chunk of the group's inputs.
template <int GS, int NM>
struct Stage {
  uint4 w[NM][GS / 32];
  float s[NM], b[NM];
  uint32_t x[RBMAX][GS / 32];
};

template <int GS, int NM, class WQ, class SB>
__device__ __forceinline__ void load_weights(Stage<GS, NM>& st, const WQ& wq, const SB& sb, int g) {
#pragma unroll
  for (int m = 0; m < NM; ++m) {
#pragma unroll
    for (int i = 0; i < GS / 32; ++i) st.w[m][i] = wq(g, m, i);
    sb(g, m, st.s[m], st.b[m]);
  }
}

// xl[r]: row r's inputs as dwords, already offset by (lane % 16)
template <int GS, int NM, int RB>
__device__ __forceinline__ void load_inputs(Stage<GS, NM>& st, const uint32_t* const (&xl)[RB], int g) {
#pragma unroll
  for (int r = 0; r < RB; ++r)
#pragma unroll
    for (int i = 0; i < GS / 32; ++i) st.x[r][i] = xl[r][(g * (GS / 32) + i) * 16];
}

template <int J, int NM, int RB>
__device__ __forceinline__ void word_dot(float (&p)[NM][RB], const uint32_t (&word)[NM], const uint32_t (&x)[RB],
                                         uint32_t magic) {
  if constexpr (J < 16) {
#pragma unroll
    for (int m = 0; m < NM; ++m) {
      constexpr int q = J & 3;
      const uint32_t b2 = and_or(q ? word[m] >> (4 * q) : word[m], NIB_MASK, magic);
#pragma unroll
      for (int r = 0; r < RB; ++r) p[m][r] = dot2_bcast<J>(p[m][r], x[r], b2);
    }
  }
}

// p += sum over chunk i of x * (128 + q)
template <int GS, int NM, int RB>
__device__ __forceinline__ void chunk_dot(float (&p)[NM][RB], const Stage<GS, NM>& st, int i) {
  const uint32_t magic = BF16_128;
  uint32_t x[RB];
#pragma unroll
  for (int r = 0; r < RB; ++r) x[r] = st.x[r][i];
#define TF_WORD(J_, C_)                                                   \
  {                                                                       \
    uint32_t word[NM];                                                    \
    _Pragma("unroll") for (int m = 0; m < NM; ++m) word[m] = st.w[m][i].C_; \
    word_dot<J_, NM, RB>(p, word, x, magic);                              \
    word_dot<J_ + 1, NM, RB>(p, word, x, magic);                          \
    word_dot<J_ + 2, NM, RB>(p, word, x, magic);                          \
    word_dot<J_ + 3, NM, RB>(p, word, x, magic);                          \
  }
  TF_WORD(0, x) TF_WORD(4, y) TF_WORD(8, z) TF_WORD(12, w)
#undef TF_WORD
}

// One wave's share of a GEMV: groups [gA, gB) of NM matrices against RB rows.
//   wq(g, m, i)     -> the lane's 16 bytes of chunk i of group g of matrix m
//   sb(g, m, s, b)  -> the lane's column's scale and bias of that group
//   xl[r]           -> row r's inputs as dwords, offset by lane % 16
//   xsum(r, g)      -> row r's sum over group g (wave-uniform)
//   flush(g, acc)   -> called after group g has been added (wave-uniform); may park and clear acc
// `st` holds the weights of groups gA .. gA + DEPTH - 1 on entry when `loaded`.
template <int GS, int NM, int RB, class WQ, class SB, class XS, class FLUSH>
__device__ __forceinline__ void gemv_stream(float (&acc)[NM][RB], Stage<GS, NM> (&st)[DEPTH], bool loaded,
                                            const WQ& wq, const SB& sb, const uint32_t* const (&xl)[RB],
                                            const XS& xsum, int gA, int gB, FLUSH& flush) {
  constexpr int CH = GS / 32;
  if (gA >= gB) return;
#pragma unroll
  for (int d = 0; d < DEPTH; ++d)
    if (gA + d < gB) {
      if (!loaded) load_weights<GS, NM>(st[d], wq, sb, gA + d);
      load_inputs<GS, NM, RB>(st[d], xl, gA + d);
    }
  for (int gb = gA; gb < gB; gb += DEPTH) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      const int g = gb + d;
      if (g < gB) {
        float p[NM][RB];
#pragma unroll
        for (int m = 0; m < NM; ++m)
#pragma unroll
          for (int r = 0; r < RB; ++r) p[m][r] = 0.f;
#pragma unroll
        for (int i = 0; i < CH; ++i) chunk_dot<GS, NM, RB>(p, st[d], i);
#pragma unroll
        for (int r = 0; r < RB; ++r) {
          const float sc = xsum(r, g);
#pragma unroll
          for (int m = 0; m < NM; ++m) {
            const float pq = fmaf(-128.f, sc, p[m][r]);
            acc[m][r] = fmaf(sc, st[d].b[m], fmaf(pq, st[d].s[m], acc[m][r]));
          }
        }
        flush(g, acc);
        if (g + DEPTH < gB) {
          load_weights<GS, NM>(st[d], wq, sb, g + DEPTH);
          load_inputs<GS, NM, RB>(st[d], xl, g + DEPTH);
        }
      }
    }
  }
}

// ---- routed experts -----------------------------------------------------------------------------------------------

__device__ __forceinline__ int slice_begin(int s, int KG) { return (int)((long long)s * KG / SLICES); }

// One pass of an item: RB of its rows (members[at0 ..]) against the workgroup's 64 columns.
// XSG: the rows' group sums come from `xs_in` (fp32 [x rows, KG], scalar loads); otherwise they are summed here
// into LDS first.  `xs_out` (may be null; epilogues 1 and 2) receives the group sums of the activations written,
// fp32 [pairs, N / GS]: what the down projection of the same pairs reads as its `xs_in`.
template <int GS, int NM, int EPI, int WAVES, int RB, bool XSG, class WQ, class SB>
__device__ __forceinline__ void expert_pass(const uint16_t* __restrict__ X, int64_t x_stride, int slots, const WQ& wq,
                                            const SB& sb, int KG, int NB, int cb2, const int* __restrict__ members,
                                            int at0, void* __restrict__ out, int N, float limit, float* xs, float* part,
                                            Stage<GS, NM> (&st)[DEPTH], bool loaded, bool first_pass,
                                            const float* __restrict__ xs_in, float* __restrict__ xs_out) {
  constexpr int SPW = SLICES / WAVES;               // slices a wave
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  int pr[RB];
  const uint16_t* xrow[RB];
  const uint32_t* xl[RB];
  const float* xsr[RB];
#pragma unroll
  for (int r = 0; r < RB; ++r) {
    pr[r] = members[at0 + r];
    const int row = slots ? pr[r] / slots : pr[r];
    xrow[r] = X + (size_t)row * x_stride;
    xl[r] = reinterpret_cast<const uint32_t*>(xrow[r]) + (lane & 15);
    xsr[r] = xs_in + (size_t)row * KG;
  }
  if (!first_pass || !XSG) __syncthreads();         // the previous pass is done with xs and part
  if constexpr (!XSG) group_sums_block<GS>(xrow, RB, KG, xs, tid, WAVES * 64);
  // slices with no group (K/gs < SLICES) still take part in the ordered sum: as zeros
  if (KG < SLICES) {
#pragma unroll
    for (int q = 0; q < SPW; ++q)
#pragma unroll
      for (int m = 0; m < NM; ++m)
#pragma unroll
        for (int r = 0; r < RB; ++r) part[(((wave * SPW + q) * NM + m) * RB + r) * 64 + lane] = 0.f;
  }
  if (!XSG || KG < SLICES) __syncthreads();
  float acc[NM][RB];
#pragma unroll
  for (int m = 0; m < NM; ++m)
#pragma unroll
    for (int r = 0; r < RB; ++r) acc[m][r] = 0.f;
  int slice = wave * SPW;
  while (slice < SLICES && slice_begin(slice + 1, KG) == slice_begin(slice, KG)) ++slice;   // skip empty slices
  int slice_end = slice < SLICES ? slice_begin(slice + 1, KG) : -1;
  auto flush = [&](int g, float (&a)[NM][RB]) {
    if (g + 1 != slice_end) return;
#pragma unroll
    for (int m = 0; m < NM; ++m)
#pragma unroll
      for (int r = 0; r < RB; ++r) {
        part[((slice * NM + m) * RB + r) * 64 + lane] = a[m][r];
        a[m][r] = 0.f;
      }
    ++slice;
    while (slice < SLICES && slice_begin(slice + 1, KG) == slice_begin(slice, KG)) ++slice;
    slice_end = slice < SLICES ? slice_begin(slice + 1, KG) : -1;
  };
  const int gA = slice_begin(wave * SPW, KG), gB = slice_begin((wave + 1) * SPW, KG);
  // with sums from memory, lane i keeps the sums of group gA + i (64 groups at a time) and readlane hands them out
  float xsv[RB];
  int xs_base = gA;
  auto fetch_sums = [&](int base) {
#pragma unroll
    for (int r = 0; r < RB; ++r) xsv[r] = base + lane < gB ? xsr[r][base + lane] : 0.f;
    xs_base = base;
  };
  if constexpr (XSG) fetch_sums(gA);
  auto xsum = [&](int r, int g) {
    if constexpr (XSG) {
      if (g - xs_base >= 64) fetch_sums(g);
      return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, xsv[r]), g - xs_base));
    } else {
      return xs[r * KG + g];
    }
  };
  gemv_stream<GS, NM, RB>(acc, st, loaded, wq, sb, xl, xsum, gA, gB, flush);
  __syncthreads();
  // a wave a row, a lane a column: the slices' sums in slice order, then the epilogue
  for (int r = wave; r < RB; r += WAVES) {
    const int l = lane;
    const int onb = 2 * cb2 + (l >> 5);
    const bool ok = onb < NB;
    float v[NM];
#pragma unroll
    for (int m = 0; m < NM; ++m) {
      float s = part[(m * RB + r) * 64 + l];
#pragma unroll
      for (int q = 1; q < SLICES; ++q) s += part[((q * NM + m) * RB + r) * 64 + l];
      v[m] = s;
    }
    int prow = pr[0];
#pragma unroll
    for (int q = 1; q < RB; ++q) prow = r == q ? pr[q] : prow;
    const size_t at = (size_t)prow * N + onb * 32 + (l & 31);
    if constexpr (EPI == 0) {
      if (ok) reinterpret_cast<float*>(out)[at] = v[0];
    } else {
      const float o = round_bf16(EPI == 1 ? relu2(v[0]) : swiglu(v[0], v[NM - 1], limit));
      if (ok) reinterpret_cast<uint16_t*>(out)[at] = (uint16_t)(__float_as_uint(o) >> 16);
      if (xs_out) {
        // group sums of the rounded activations: a fixed xor tree over the group's lanes
        float t = ok ? o : 0.f;
#pragma unroll
        for (int m = 1; m < GS; m <<= 1) t += __shfl_xor(t, m);
        if (ok && (l & (GS - 1)) == 0) xs_out[(size_t)prow * (N / GS) + (cb2 * 64 + l) / GS] = t;
      }
    }
  }
}

// A workgroup takes (item, pair of 32-column blocks): lanes 0-31 the even block, lanes 32-63 the odd one.
// Pair p reads X row p / slots when slots > 0, else row p (experts.cu:129).  The item's rows go through in passes
// of 2 or 1; a row's arithmetic is the same in each, so its bits do not depend on the pass it lands in.
template <int GS, int NM, int EPI, int WAVES, bool XSG>
__global__ void __launch_bounds__(WAVES * 64)
    expert_kernel(const uint16_t* __restrict__ X, int64_t x_stride, int slots, const uint32_t* __restrict__ W, int KG,
                  int NB, const int* __restrict__ items, const int* __restrict__ counts,
                  const int* __restrict__ members, void* __restrict__ out, int N, float limit,
                  const float* __restrict__ xs_in, float* __restrict__ xs_out) {
  constexpr int BW = block_words(GS);
  constexpr int SPW = SLICES / WAVES;
  extern __shared__ float lds[];            // xs [RBMAX][KG], then the slices' sums [SLICES][NM][RBMAX][64]
  const int NB2 = (NB + 1) >> 1;
  const int it = blockIdx.x / NB2, cb2 = blockIdx.x - it * NB2;
#ifdef TF_X_FAKEITEM
  if (it >= 41) return;
  const int e = (it * 3) & 127, first = it, cnt = 1;
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
  const int gA = slice_begin(wave * SPW, KG), gB = slice_begin((wave + 1) * SPW, KG);
  float* xs = lds;
  float* part = lds + (XSG ? 0 : RBMAX * KG);
  // the wave's first groups are on their way before anything else is read
  Stage<GS, NM> st[DEPTH];
#pragma unroll
  for (int d = 0; d < DEPTH; ++d)
    if (gA + d < gB) load_weights<GS, NM>(st[d], wq, sb, gA + d);
  bool loaded = true, first_pass = true;
  int r0 = 0;
#define TF_PASS(RB_)                                                                                                 \
  expert_pass<GS, NM, EPI, WAVES, RB_, XSG>(X, x_stride, slots, wq, sb, KG, NB, cb2, members, first + r0, out, N,    \
                                            limit, xs, part, st, loaded, first_pass, xs_in, xs_out);                 \
  first_pass = false;                                                                                                \
  loaded = gB - gA <= DEPTH   /* a run that fits the stages stays in registers for the next pass */
  for (; r0 + 2 <= cnt; r0 += 2) {
    TF_PASS(2);
  }
  if (r0 < cnt) {
    TF_PASS(1);
  }
#undef TF_PASS
}

// ---- dense lane matmul ---------------------------------------------------------------------------------------------

struct NoFlush {
  template <class A>
  __device__ __forceinline__ void operator()(int, A&) const {}
};

// One pass of a row tile: RB rows r0 .. r0 + RB - 1 against the workgroup's 64 columns and K slice.
template <int GS, int WAVES, int RB, class WQ, class SB>
__device__ __forceinline__ void qmm_pass(const uint16_t* __restrict__ X, int64_t ldx, const float* __restrict__ XS,
                                         const WQ& wq, const SB& sb, int r0, int tile, int slice, int gs0, int per,
                                         int g0, int g1, void* __restrict__ out, float* __restrict__ part_out, int M,
                                         int N, int KG, int SK, int f32, float* xs, float* part,
                                         Stage<GS, 1> (&st)[DEPTH], bool loaded) {
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const uint32_t* xl[RB];
  const_u32_ptr xsr[RB];
#pragma unroll
  for (int r = 0; r < RB; ++r) {
    xl[r] = reinterpret_cast<const uint32_t*>(X + (size_t)(r0 + r) * ldx) + (lane & 15);
    xsr[r] = as_const(XS + (size_t)(r0 + r) * KG);
  }
  __syncthreads();                                  // the previous pass is done with part
  float acc[1][RB];
#pragma unroll
  for (int r = 0; r < RB; ++r) acc[0][r] = 0.f;
  NoFlush none;
  auto xsum = [&](int r, int g) { return __uint_as_float(xsr[r][g]); };
  gemv_stream<GS, 1, RB>(acc, st, loaded, wq, sb, xl, xsum, g0, g1, none);
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
// split them again (added in wave order); SK > 1 leaves the slice's fp32 sums in part[z].  Rows go in passes of 2 or 1.
template <int GS, int WAVES>
__global__ void __launch_bounds__(WAVES * 64)
    qmm_kernel(const uint16_t* __restrict__ X, int64_t ldx, const float* __restrict__ XS,
               const uint32_t* __restrict__ W, const uint16_t* __restrict__ S, const uint16_t* __restrict__ B,
               int64_t sb_stride, void* __restrict__ out, float* __restrict__ part_out, int M, int N, int KG, int SK,
               int BM, int f32) {
  extern __shared__ float lds[];            // partials [WAVES][RBMAX][64]
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
  float* xs = nullptr;
  float* part = lds;
  const int m_end = min(M, (rt + 1) * BM);
  int r0 = rt * BM;
  Stage<GS, 1> st[DEPTH];
#pragma unroll
  for (int d = 0; d < DEPTH; ++d)
    if (g0 + d < g1) load_weights<GS, 1>(st[d], wq, sb, g0 + d);
  bool loaded = true;
#define TF_QMM_PASS(RB_)                                                                                             \
  qmm_pass<GS, WAVES, RB_>(X, ldx, XS, wq, sb, r0, tile, slice, gs0, per, g0, g1, out, part_out, M, N, KG, SK, f32, xs, \
                           part, st, loaded);                                                                        \
  loaded = g1 - g0 <= DEPTH
  for (; r0 + 2 <= m_end; r0 += 2) {
    TF_QMM_PASS(2);
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

constexpr int QMM_WAVES = 4;

// Waves a workgroup of the expert GEMV: few workgroups (a small batch) spread each one's K over 16 waves, many
// workgroups keep 4 longer-running waves each so that more of them are resident.  Scheduling only: bits do not move.
int expert_waves(int64_t grid) {
  static const int forced = [] {
    const char* v = getenv("TENSORFOLD_AMD_EXPERT_WAVES");
    return v ? atoi(v) : 0;
  }();
  if (forced == 4 || forced == 8 || forced == 16) return forced;
  return grid < 384 ? 16 : grid < 768 ? 8 : 4;
}

template <int GS, int NM, int EPI, bool XSG>
int launch_experts(const uint16_t* x, int64_t x_stride, int slots, const uint32_t* w, int kg, int nb, const int* items,
                   const int* counts, const int* members, void* out, int n, float limit, int64_t max_units,
                   const float* xs_in, float* xs_out, hipStream_t stream) {
  const int nb2 = (nb + 1) / 2;
  const int64_t max_items = (max_units + nb - 1) / nb;
  const int64_t grid = max_items * nb2;
  if (grid < 1) return 0;
  TF_REQUIRE(grid <= 0x7FFFFFFF, "experts: %lld workgroups exceed the grid limit", (long long)grid);
  const size_t smem = sizeof(float) * ((XSG ? 0 : (size_t)RBMAX * kg) + (size_t)SLICES * NM * RBMAX * 64);
  TF_REQUIRE(smem <= 64 * 1024, "experts: K/gs = %d groups need %zu bytes of LDS (limit 65536)", kg, smem);
  const dim3 g((unsigned)grid);
#define TF_GO(W_)                                                                                                  \
  expert_kernel<GS, NM, EPI, W_, XSG><<<g, W_ * 64, smem, stream>>>(x, x_stride, slots, w, kg, nb, items, counts, \
                                                                    members, out, n, limit, xs_in, xs_out)
  switch (expert_waves(grid)) {
    case 16: TF_GO(16); break;
    case 8: TF_GO(8); break;
    default: TF_GO(4);
  }
#undef TF_GO
  TF_LAUNCH_OK("tf_experts_run");
  return 0;
}

}  // namespace
}  // namespace tf

using namespace tf;

extern "C" int tf_experts_run(int gs, int epi, const uint16_t* x, int64_t x_stride, int slots, const uint32_t* w,
                              int kg, int nb, const int32_t* items, const int32_t* counts, const int32_t* members,
                              void* out, int n, float limit, int64_t max_units, const float* xs, float* xs_out,
                              tf_stream_t stream) {
  clear_error();
  TF_REQUIRE(gs == 32 || gs == 64, "experts: groups of 32 or 64 inputs, not %d", gs);
  TF_REQUIRE(x && w && items && counts && members && out, "experts: null pointer argument");
  TF_REQUIRE(!xs_out || (epi != 0 && n % gs == 0), "experts: xs_out goes with an activation epilogue and whole groups");
  TF_REQUIRE(kg >= 1 && nb >= 1 && n == nb * 32, "experts: n (%d) must be the column blocks (%d) times 32", n, nb);
  TF_REQUIRE(aligned16(x) && x_stride % 8 == 0, "x: rows of K = groups * group size inputs, 16-byte aligned");
  TF_REQUIRE(aligned16(w), "w must be 16-byte aligned");
  TF_REQUIRE(slots >= 0 && max_units >= 0, "experts: negative slots or max_units");
  hipStream_t s = as_stream(stream);
#define TF_RUN(GS_, NM_, EPI_)                                                                                       \
  if (gs == GS_ && epi == EPI_)                                                                                      \
    return xs ? launch_experts<GS_, NM_, EPI_, true>(x, x_stride, slots, w, kg, nb, items, counts, members, out, n,  \
                                                     limit, max_units, xs, xs_out, s)                                \
              : launch_experts<GS_, NM_, EPI_, false>(x, x_stride, slots, w, kg, nb, items, counts, members, out, n, \
                                                      limit, max_units, xs, xs_out, s);
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
  const size_t smem = sizeof(float) * ((size_t)QMM_WAVES * RBMAX * 64);
  TF_REQUIRE((int64_t)tiles * rts <= 0x7FFFFFFF && sk <= 65535, "qmm: grid too large");
  const dim3 grid((unsigned)(tiles * rts), 1, (unsigned)sk);
  if (gs == 64)
    qmm_kernel<64, QMM_WAVES><<<grid, QMM_WAVES * 64, smem, s>>>(x, ldx, xs, weight, scales, biases, sb_stride, out,
                                                                part, m, n, kg, sk, bm, f32);
  else
    qmm_kernel<32, QMM_WAVES><<<grid, QMM_WAVES * 64, smem, s>>>(x, ldx, xs, weight, scales, biases, sb_stride, out,
                                                                part, m, n, kg, sk, bm, f32);
  TF_LAUNCH_OK("tf_qmm");
  if (sk > 1 && reduce) {
    const long long total = (long long)m * n;
    qmm_reduce_kernel<<<(unsigned)((total + 255) / 256), 256, 0, s>>>(part, out, total, sk, f32);
    TF_LAUNCH_OK("tf_qmm reduce");
  }
  return 0;
}
