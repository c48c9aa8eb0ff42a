// The decode-form GEMV core shared by the stand-alone expert and lane kernels (decode.hip) and the fused MoE layer
// (fused.hip): one wave's streaming loop, the per-item pass with its ordered K-slice sums and epilogues.
#pragma once

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
  const u32x4_t v = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(p));
  return make_uint4(v.x, v.y, v.z, v.w);
}

// (x & mask) | magic in one VALU op; the mask rides in an SGPR and the magic in a VGPR (one constant-bus read)
__device__ __forceinline__ uint32_t and_or(uint32_t x, uint32_t mask, uint32_t magic) {
  uint32_t r;
  asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(x), "s"(mask), "v"(magic));
  return r;
}

// Agent-scope relaxed accesses: coherent across the chip's L2s (sc1) without any cache-wide write-back or
// invalidate.  The fused layer moves its activations between workgroups through them.
template <class T>
__device__ __forceinline__ T ld_agent(const T* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
template <class T>
__device__ __forceinline__ void st_agent(T* p, T v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
constexpr int COH_IN = 1, COH_OUT = 2;     // which side of a unit goes through agent-scope accesses

constexpr int SLICES = 16;      // K slices of the expert GEMV
constexpr int DEPTH = 2;        // groups of weights a wave keeps in flight
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
// the lane's dword of each chunk of the group's inputs.  Scale and bias stay as they were loaded (bf16 bits: the
// scale in the low half of `s`, the bias in the low half of `b`, or with BHI in its high half) until the group is
// added: turning them into floats where they are loaded would make the wave wait for every load it has just issued.
// RBM: the most rows a pass of the kernel holding the stage takes.
template <int GS, int NM, int RBM = RBMAX>
struct Stage {
  uint4 w[NM][GS / 32];
  uint32_t s[NM], b[NM];
  uint32_t x[RBM][GS / 32];
};

template <int GS, int NM, int RBM, class WQ, class SB>
__device__ __forceinline__ void load_weights(Stage<GS, NM, RBM>& st, const WQ& wq, const SB& sb, int g) {
#pragma unroll
  for (int m = 0; m < NM; ++m) {
#pragma unroll
    for (int i = 0; i < GS / 32; ++i) st.w[m][i] = wq(g, m, i);
    sb(g, m, st.s[m], st.b[m]);
  }
}

// The sum of a row of 16 lanes, left in every one of them: the two quad swaps, then the mirrored halves of 8 and of
// 16 lanes.  Both sides of each step add the same two numbers, so all sixteen lanes end with the same bits.
__device__ __forceinline__ float row16_sum(float s) {
#define TF_DPP_ADD(CTRL_) \
  s += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, s), CTRL_, 0xF, 0xF, true))
  TF_DPP_ADD(0xB1);        // quad_perm [1, 0, 3, 2]
  TF_DPP_ADD(0x4E);        // quad_perm [2, 3, 0, 1]
  TF_DPP_ADD(0x141);       // row_half_mirror
  TF_DPP_ADD(0x140);       // row_mirror
#undef TF_DPP_ADD
  return s;
}

// Row r's sum over the staged group, from the dwords the dot products read anyway: a lane adds its two inputs of
// each chunk in chunk order (a dot product against ones), then the sixteen lanes that share the row add up.
template <int GS, int NM, int RBM>
__device__ __forceinline__ float stage_row_sum(const Stage<GS, NM, RBM>& st, int r) {
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < GS / 32; ++i) s = dot2(st.x[r][i], BF16_ONES, s);
  return row16_sum(s);
}

// xl[r]: row r's inputs as dwords, already offset by (lane % 16)
template <int GS, int NM, int RB, int COH, int RBM>
__device__ __forceinline__ void load_inputs(Stage<GS, NM, RBM>& st, const uint32_t* const (&xl)[RB], int g) {
#pragma unroll
  for (int r = 0; r < RB; ++r)
#pragma unroll
    for (int i = 0; i < GS / 32; ++i) {
      const uint32_t* p = xl[r] + (g * (GS / 32) + i) * 16;
      st.x[r][i] = (COH & COH_IN) ? ld_agent(p) : *p;
    }
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
template <int GS, int NM, int RB, int RBM>
__device__ __forceinline__ void chunk_dot(float (&p)[NM][RB], const Stage<GS, NM, RBM>& st, int i) {
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

// A group's term by itself: fma(xs, b, P s), the product rounded once before the bias term joins it.
__device__ __forceinline__ float group_term(float pq, float scale, float sc, float bias) {
  return fmaf(sc, bias, __fmul_rn(pq, scale));
}

// One wave's share of a GEMV: groups [gA, gB) of NM matrices against RB rows.
//   wq(g, m, i)     -> the lane's 16 bytes of chunk i of group g of matrix m
//   sb(g, m, s, b)  -> the lane's column's scale and bias of that group, as loaded (see Stage)
//   xl[r]           -> row r's inputs as dwords, offset by lane % 16
//   xsum(r, g)      -> row r's sum over group g (wave-uniform); with XIN the sums are taken from the staged inputs
//   flush(g, acc)   -> called after group g has been added (wave-uniform); may park and clear acc
// `st` holds the weights of groups gA .. gA + DEPTH - 1 on entry when `loaded`.
// SEPG: a group's term is rounded by itself, t = fma(xs, b, P s), and added to the running sum (acc + t) instead of
// being chained through it.  The down projection of the routed experts sums this way, so that a kernel that holds one
// group of an expert's inputs (the decode layer cut along the intermediate width) can leave t for another workgroup
// to add and arrive at the same bits.
template <int GS, int NM, int RB, int COH, bool XIN = false, bool BHI = false, bool SEPG = false, int RBM, class WQ,
          class SB, class XS, class FLUSH>
__device__ __forceinline__ void gemv_stream(float (&acc)[NM][RB], Stage<GS, NM, RBM> (&st)[DEPTH], bool loaded,
                                            const WQ& wq, const SB& sb, const uint32_t* const (&xl)[RB],
                                            const XS& xsum, int gA, int gB, FLUSH& flush) {
  constexpr int CH = GS / 32;
  if (gA >= gB) return;
#pragma unroll
  for (int d = 0; d < DEPTH; ++d)
    if (gA + d < gB) {
      if (!loaded) load_weights<GS, NM>(st[d], wq, sb, gA + d);
      load_inputs<GS, NM, RB, COH>(st[d], xl, gA + d);
    }
  const int n = gB - gA;
  for (int gb = gA; gb < gB; gb += DEPTH) {
    if (n > DEPTH) prio_by_progress(gB - gb, n);      // (one trip through this loop: nobody to yield to)
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
        // A dot instruction's result may be read by a different VALU instruction only three wait states later;
        // the compiler inserts them for instructions it emits itself, not after inline assembly.
#pragma unroll
        for (int m = 0; m < NM; ++m)
#pragma unroll
          for (int r = 0; r < RB; ++r) asm volatile("s_nop 2" : "+v"(p[m][r]));
#pragma unroll
        for (int r = 0; r < RB; ++r) {
          float sc;
          if constexpr (XIN) sc = stage_row_sum<GS, NM>(st[d], r);
          else sc = xsum(r, g);
#pragma unroll
          for (int m = 0; m < NM; ++m) {
            const float pq = fmaf(-128.f, sc, p[m][r]);
            const float scale = __uint_as_float(st[d].s[m] << 16);
            const float bias = __uint_as_float(BHI ? st[d].b[m] & 0xFFFF0000u : st[d].b[m] << 16);
            if constexpr (SEPG) acc[m][r] = __fadd_rn(acc[m][r], group_term(pq, scale, sc, bias));
            else acc[m][r] = fmaf(sc, bias, fmaf(pq, scale, acc[m][r]));
          }
        }
        flush(g, acc);
        if (g + DEPTH < gB) {
          load_weights<GS, NM>(st[d], wq, sb, g + DEPTH);
          load_inputs<GS, NM, RB, COH>(st[d], xl, g + DEPTH);
        }
      }
    }
  }
}

// ---- routed experts -----------------------------------------------------------------------------------------------

__device__ __forceinline__ int slice_begin(int s, int KG) { return (int)((long long)s * KG / SLICES); }

// What a caller may hang on a unit (see expert_unit): `streamed()` runs in every wave once it has issued the last of
// its own loads and before the workgroup meets to add the slices up; `act(r, l, bits)` receives the bf16 bits of
// activation column l (of the unit's 64) of row r when the epilogue makes activations.
struct NoSink {
  __device__ __forceinline__ void streamed() const {}
  __device__ __forceinline__ void act(int, int, uint32_t) const {}
};

// One pass of an item: RB of its rows (pairs[0 ..]) against the workgroup's 64 columns.
// Each wave takes the sums of its groups' inputs from the dwords it reads for the dot products.
template <int GS, int NM, int EPI, int WAVES, int RB, int COH, class WQ, class SB, class SINK>
__device__ __forceinline__ void expert_pass(const uint16_t* __restrict__ X, int64_t x_stride, int slots, const WQ& wq,
                                            const SB& sb, int KG, int NB, int cb2, const int* pairs,
                                            void* __restrict__ out, int N, float limit, float* part,
                                            Stage<GS, NM> (&st)[DEPTH], bool loaded, bool first_pass, SINK& sink) {
  constexpr int SPW = SLICES / WAVES;               // slices a wave
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  int pr[RB];
  const uint16_t* xrow[RB];
  const uint32_t* xl[RB];
#pragma unroll
  for (int r = 0; r < RB; ++r) {
    pr[r] = pairs[r];
    const int row = slots ? pr[r] / slots : pr[r];
    xrow[r] = X + (size_t)row * x_stride;
    xl[r] = reinterpret_cast<const uint32_t*>(xrow[r]) + (lane & 15);
  }
  if (!first_pass) __syncthreads();                 // the previous pass is done with part
  // slices with no group (K/gs < SLICES) still take part in the ordered sum: as zeros
  if (KG < SLICES) {
#pragma unroll
    for (int q = 0; q < SPW; ++q)
#pragma unroll
      for (int m = 0; m < NM; ++m)
#pragma unroll
        for (int r = 0; r < RB; ++r) part[(((wave * SPW + q) * NM + m) * RB + r) * 64 + lane] = 0.f;
  }
  if (KG < SLICES) __syncthreads();
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
  auto no_sums = [](int, int) { return 0.f; };
  if (first_pass) TF_MARK(2);
  // the down projection (EPI 0) adds each group's term by itself: see gemv_stream
  gemv_stream<GS, NM, RB, COH, true, true, EPI == 0>(acc, st, loaded, wq, sb, xl, no_sums, gA, gB, flush);
  TF_MARK(3);
  sink.streamed();
  __syncthreads();
  TF_MARK(4);
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
      if (ok) {
        if (COH & COH_OUT) st_agent(reinterpret_cast<float*>(out) + at, v[0]);
        else reinterpret_cast<float*>(out)[at] = v[0];
      }
    } else {
      const float o = round_bf16(EPI == 1 ? relu2(v[0]) : swiglu(v[0], v[NM - 1], limit));
      const uint32_t bits = __float_as_uint(o) >> 16;
      sink.act(r, l, ok ? bits : 0u);
      if (COH & COH_OUT) {
        // two columns a dword, written by the even lane (N is even, rows are dword-aligned)
        const uint32_t hi = __shfl_down(bits, 1);
        if (ok && !(l & 1)) st_agent(reinterpret_cast<uint32_t*>(reinterpret_cast<uint16_t*>(out) + at), bits | (hi << 16));
      } else if (ok) {
        reinterpret_cast<uint16_t*>(out)[at] = (uint16_t)bits;
      }
    }
  }
}

struct NoHook {
  __device__ __forceinline__ bool operator()() const { return true; }
};

// (item, pair of 32-column blocks) of one expert matrix set: lanes 0-31 take the even block, lanes 32-63 the odd one.
// Pair p reads X row p / slots when slots > 0, else row p (experts.cu:129 of the reference).  The item's rows go
// through in passes of 2 or 1; a row's arithmetic is the same in each, so its bits do not depend on the pass it
// lands in.  `ready()` runs after the wave's first weights have been requested and before any activation is read
// (the fused layer waits there for the item's activations); returning false abandons the unit.
// lds: the slices' sums [SLICES][NM][RBMAX][64].
template <int GS, int NM, int EPI, int WAVES, int COH, class HOOK, class SINK = NoSink>
__device__ __forceinline__ bool expert_unit(const uint16_t* __restrict__ X, int64_t x_stride, int slots,
                                            const uint32_t* __restrict__ W, int KG, int NB, int e, int cnt,
                                            const int* pairs, int cb2, void* __restrict__ out, int N, float limit,
                                            float* lds, HOOK& ready, SINK&& sink = SINK()) {
  constexpr int BW = block_words(GS);
  constexpr int SPW = SLICES / WAVES;
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int nb = 2 * cb2 + (lane >> 5), c = lane & 31;
  const bool col_ok = nb < NB;
  const uint32_t* wbase =
      W + (((size_t)e * NB + (col_ok ? nb : NB - 1)) * KG) * (size_t)(NM * BW) + c * 4;
  const uint32_t* sbase = wbase - c * 4 + 32 * GS / 8 + c;
  auto wq = [&](int g, int m, int i) { return ldg16(wbase + ((size_t)g * NM + m) * BW + i * 128); };
  auto sb = [&](int g, int m, uint32_t& s, uint32_t& b) {
    s = b = __builtin_nontemporal_load(sbase + ((size_t)g * NM + m) * BW);      // (scale | bias << 16)
  };
  TF_MARK(1);
  const int gA = slice_begin(wave * SPW, KG), gB = slice_begin((wave + 1) * SPW, KG);
  float* part = lds;
  // the wave's first groups are on their way before anything else is read
  Stage<GS, NM> st[DEPTH];
#pragma unroll
  for (int d = 0; d < DEPTH; ++d)
    if (gA + d < gB) load_weights<GS, NM>(st[d], wq, sb, gA + d);
  if (!ready()) return false;
  bool loaded = true, first_pass = true;
  int r0 = 0;
#define TF_PASS(RB_)                                                                                                \
  expert_pass<GS, NM, EPI, WAVES, RB_, COH>(X, x_stride, slots, wq, sb, KG, NB, cb2, pairs + r0, out, N, limit, part, \
                                            st, loaded, first_pass, sink);                                          \
  first_pass = false;                                                                                               \
  loaded = gB - gA <= DEPTH   /* a run that fits the stages stays in registers for the next pass */
  for (; r0 + 2 <= cnt; r0 += 2) {
    TF_PASS(2);
  }
  if (r0 < cnt) {
    TF_PASS(1);
  }
#undef TF_PASS
  TF_MARK(5);
  return true;
}

// LDS floats a workgroup of expert_unit needs
constexpr size_t expert_lds_floats(int nm) { return (size_t)SLICES * nm * RBMAX * 64; }

}  // namespace
}  // namespace tf
