// EXL3 trellis decode shared by the dense linear and the routed experts: window extraction, codebooks, the
// 128-point Hadamard butterfly, and one wave's decode-and-MFMA walk over a 128-column block.
//
// A tile holds 256 values of k2/2 bits in a circular bitstream (most significant bit of each little-endian 32-bit
// word first); value p is the 16-bit window ending at bit E(p), pushed through a procedural codebook to an fp16
// value, and lands at row 2 (l % 4) + (j & 1) + 8 ((j >> 1) & 1), column l / 4 + 8 (j >> 2) of the 16 x 16 tile
// (l = p / 8, j = p % 8)  (reference: docs/recipes/exl3.md:43-63, cuda/exl3/format.py:31-110).
//
// On a 64-lane wave the B operand of v_mfma_f32_16x16x32_f16 is 32 inputs x 16 columns, 8 values a lane: lane
// (column c, quarter kq) takes, from each of two consecutive k tiles, the four stream-consecutive values
// p0 .. p0 + 3 with p0 = 8 (4 (c % 8) + kq) + 4 (c / 8).  They sit in rows {2 kq, 2 kq + 1, 2 kq + 8, 2 kq + 9} of
// column c, so the A operand reads the rotated activations at the same eight inputs and no value moves across
// lanes.  Rows of the call are MFMA rows: independent by construction.  K is split over waves and blocks as a
// function of the shape only and every sum runs in a fixed order.


#ifndef TF_EXL3_DECODE_H
#define TF_EXL3_DECODE_H

#include <hip/hip_fp16.h>

#include "tf_common.h"

namespace tf {
namespace {

constexpr float HAD_SCALE = 0.08838834764831845f;   // 1 / sqrt(128)

template <int K2>
__host__ __device__ constexpr int tile_words() {
  return 4 * K2;
}

// E(p): one past the last stream bit of value p's window
template <int K2>
__host__ __device__ constexpr int stream_end(int p) {
  return (K2 & 1) ? ((p + 1) * K2 - ((p + 1) & 1)) / 2 : (p + 1) * (K2 / 2);
}

// bit distance from value p0's window to value p0 + j's, p0 a multiple of 4
template <int K2>
__host__ __device__ constexpr int delta(int j) {
  return stream_end<K2>(j) - stream_end<K2>(0);
}

// The stored words lane (L, h) needs of a tile for its four values p0 .. p0 + 3 (p0 = 8 L + 4 h): two, or three when
// a window can reach past the second.
template <int K2>
struct Windows {
  static constexpr int TW = tile_words<K2>(), R = 32 * TW;
  static constexpr bool NEED_LO = delta<K2>(3) + 16 > 32;      // a window reaches past the first aligned word
  static constexpr bool NEED_W2 = 31 + delta<K2>(3) + 16 > 64; // ... and past the second stored word
  static constexpr int NW = NEED_LO && NEED_W2 ? 3 : 2;
  int wi, wi1, wi2, o;                                         // the words and the bit offset: the same for every tile
  __device__ __forceinline__ Windows(int L, int h) {
    const int p0 = 8 * L + 4 * h;
    const int first = (stream_end<K2>(0) + p0 * K2 / 2 - 16 + R) % R;   // E(p0) - 16; p0 is even, p0 * K2 / 2 whole
    wi = first >> 5;
    wi1 = (wi + 1) % TW;
    wi2 = (wi + 2) % TW;
    o = first & 31;
  }
  __device__ __forceinline__ void load(const uint32_t* tile, uint32_t (&w)[NW]) const {
    w[0] = tile[wi];
    w[1] = tile[wi1];
    if constexpr (NW == 3) w[2] = tile[wi2];
  }
  // the 16-bit states of the four values
  __device__ __forceinline__ void states(const uint32_t (&w)[NW], uint32_t (&s)[4]) const {
    const uint32_t hi = __funnelshift_l(w[1], w[0], o);        // the stream from the first window on, 32 bits
    uint32_t lo = 0;
    if constexpr (NEED_LO) lo = __funnelshift_l(NW == 3 ? w[NW - 1] : 0u, w[1], o);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int d = delta<K2>(j);
      if (d + 16 <= 32) s[j] = (hi >> (16 - d)) & 0xFFFFu;
      else if (d < 32) s[j] = __funnelshift_l(lo, hi, d) >> 16;
      else s[j] = (lo >> (48 - d)) & 0xFFFFu;
    }
  }
};

// fp16 bits of the codebook value of state s
template <int CB>
__device__ __forceinline__ uint16_t code_value(uint32_t s) {
  if constexpr (CB == 2) {
    const uint32_t x = s * 0x83DCD12Du;
    const uint32_t hs = 1024u + (x & 255u) + ((x >> 8) & 255u) + ((x >> 16) & 255u) + (x >> 24);
    const __half hv = __ushort_as_half((unsigned short)(0x6400u + (hs - 1024u)));   // fp16 of 1024 + byte sum (< 2048)
    const __half r = __hfma(hv, __ushort_as_half((unsigned short)0x1EEE), __ushort_as_half((unsigned short)0xC931));
    return __half_as_ushort(r);
  } else {
    uint32_t x = CB == 1 ? s * 0xCBAC1FEDu : s * 89226354u + 64248484u;
    x = (x & 0x8FFF8FFFu) ^ 0x3B603B60u;
    const __half r = __hadd(__ushort_as_half((unsigned short)(x & 0xFFFFu)), __ushort_as_half((unsigned short)(x >> 16)));
    return __half_as_ushort(r);
  }
}

// The hashed word of a state of the 3inst and mcg codebooks: the value is the fp16 sum of its two halves.
template <int CB>
__device__ __forceinline__ uint32_t code_word(uint32_t s) {
  const uint32_t x = CB == 1 ? s * 0xCBAC1FEDu : s * 89226354u + 64248484u;
  return (x & 0x8FFF8FFFu) ^ 0x3B603B60u;
}

// (half(xa.lo) + half(xa.hi)) | (half(xb.lo) + half(xb.hi)) << 16.  The second add writes the upper half of the
// register the first one wrote and keeps the lower: two instructions for two values, where the compiler's own
// pairing pads each result and ORs them (a third).  The same IEEE add as __hadd.
__device__ __forceinline__ uint32_t half_sums(uint32_t xa, uint32_t xb) {
  uint32_t r;
  asm("v_add_f16_sdwa %0, %1, %1 dst_sel:WORD_0 dst_unused:UNUSED_PAD src0_sel:WORD_0 src1_sel:WORD_1" : "=v"(r) : "v"(xa));
  asm("v_add_f16_sdwa %0, %1, %1 dst_sel:WORD_1 dst_unused:UNUSED_PRESERVE src0_sel:WORD_0 src1_sel:WORD_1"
      : "+v"(r)
      : "v"(xb));
  return r;
}

// the fp16 bits of the lane's four values of one tile, as two packed words
template <int K2, int CB>
__device__ __forceinline__ void decode4(const Windows<K2>& win, const uint32_t (&w)[Windows<K2>::NW], uint32_t& lo,
                                        uint32_t& hi) {
  uint32_t s[4];
  win.states(w, s);
  if constexpr (CB == 2) {
    lo = (uint32_t)code_value<CB>(s[0]) | ((uint32_t)code_value<CB>(s[1]) << 16);
    hi = (uint32_t)code_value<CB>(s[2]) | ((uint32_t)code_value<CB>(s[3]) << 16);
  } else {
    lo = half_sums(code_word<CB>(s[0]), code_word<CB>(s[1]));
    hi = half_sums(code_word<CB>(s[2]), code_word<CB>(s[3]));
  }
}

template <int K2, int CB>
__device__ __forceinline__ void values4(const uint32_t* tile, int L, int h, uint16_t (&v)[4]) {
  const Windows<K2> win(L, h);
  uint32_t w[Windows<K2>::NW], lo, hi;
  win.load(tile, w);
  decode4<K2, CB>(win, w, lo, hi);
  v[0] = (uint16_t)lo;
  v[1] = (uint16_t)(lo >> 16);
  v[2] = (uint16_t)hi;
  v[3] = (uint16_t)(hi >> 16);
}

// Unscaled Walsh-Hadamard transform of 128 values, two a lane (elements 2 lane, 2 lane + 1), fixed butterfly order.
__device__ __forceinline__ void fwht128(float& a, float& b, int lane) {
  const float s = a + b, d = a - b;
  a = s;
  b = d;
#pragma unroll
  for (int m = 1; m < 64; m <<= 1) {
    const float oa = __shfl_xor(a, m), ob = __shfl_xor(b, m);
    a = (lane & m) ? oa - a : a + oa;
    b = (lane & m) ? ob - b : b + ob;
  }
}

__device__ __forceinline__ void load2(const void* p, int dtype, size_t i, float& a, float& b) {
  if (dtype == TF_F32) {
    const float2 u = *reinterpret_cast<const float2*>(static_cast<const float*>(p) + i);
    a = u.x;
    b = u.y;
  } else if (dtype == TF_BF16) {
    const uint32_t u = *reinterpret_cast<const uint32_t*>(static_cast<const uint16_t*>(p) + i);
    a = bf16_lo(u);
    b = bf16_hi(u);
  } else {
    const __half2 u = *reinterpret_cast<const __half2*>(static_cast<const __half*>(p) + i);
    a = __low2float(u);
    b = __high2float(u);
  }
}

__device__ __forceinline__ void store2(void* p, int dtype, size_t i, float a, float b) {
  if (dtype == TF_F32) {
    *reinterpret_cast<float2*>(static_cast<float*>(p) + i) = make_float2(a, b);
  } else if (dtype == TF_BF16) {
    *reinterpret_cast<uint32_t*>(static_cast<uint16_t*>(p) + i) = pack_bf16(a, b);
  } else {
    *reinterpret_cast<__half2*>(static_cast<__half*>(p) + i) = __floats2half2_rn(a, b);
  }
}


// The lane's two columns' output scales and bias of a layer, loaded once for all the rows a wave finishes.
struct OutScale {
  float sa, sb, ba, bb;
  __device__ __forceinline__ OutScale(const uint16_t* svh, const uint16_t* bias, int col) {
    load2(svh, TF_F16, col, sa, sb);
    ba = bb = 0.f;
    has_bias = bias != nullptr;
    if (bias) load2(bias, TF_F16, col, ba, bb);
  }
  bool has_bias;
};

// the finished outputs of one row's 128 columns from their fp32 sums: H / sqrt(128), * svh, + bias
__device__ __forceinline__ void finish_values(float& a, float& b, int lane, const OutScale& s) {
  fwht128(a, b, lane);
  a = a * HAD_SCALE * s.sa;
  b = b * HAD_SCALE * s.sb;
  if (s.has_bias) {
    a += s.ba;
    b += s.bb;
  }
}

__device__ __forceinline__ void finish_row(float a, float b, int lane, const OutScale& s, void* y, int y_dtype,
                                           size_t at) {
  finish_values(a, b, lane, s);
  store2(y, y_dtype, at, a, b);
}

__device__ __forceinline__ void finish_row(float a, float b, int lane, const uint16_t* svh, const uint16_t* bias,
                                           int col, void* y, int y_dtype, size_t at) {
  finish_row(a, b, lane, OutScale(svh, bias, col), y, y_dtype, at);
}

// a value as a store to `dtype` and a load back leave it
__device__ __forceinline__ float rounded(float v, int dtype) {
  if (dtype == TF_F32) return v;
  if (dtype == TF_BF16) return round_bf16(v);
  return __half2float(__float2half_rn(v));
}

// SwiGLU of one row's 128 columns of gate (g) and up (u), two a lane, then the next layer's input rotation with its
// input scales (sa, sb): xh[at ..] = fp16(((act * suh) H) / sqrt(128)).  g and u are rounded to `dtype` first (what a
// y of that type holds), act = rounded(rounded(g / (1 + exp(-g))) * u): the roundings of the two elementwise steps
// on tensors of that type.
__device__ __forceinline__ void swiglu_rot(float g0, float g1, float u0, float u1, int dtype, int lane, float sa,
                                           float sb, uint16_t* xh, size_t at) {
  g0 = rounded(g0, dtype), g1 = rounded(g1, dtype), u0 = rounded(u0, dtype), u1 = rounded(u1, dtype);
  float a = rounded(rounded(g0 / (1.f + expf(-g0)), dtype) * u0, dtype);
  float b = rounded(rounded(g1 / (1.f + expf(-g1)), dtype) * u1, dtype);
  a *= sa;
  b *= sb;
  fwht128(a, b, lane);
  store2(xh, TF_F16, at, a * HAD_SCALE, b * HAD_SCALE);
}

// One wave's sums of up to 16 rows over the k-tile pairs [pr0, pr1) of a 128-column block: acc[j] is the 16 x 16
// tile of column tile j.  xr: the lane's A row (row c of the pass) + 2 kq; stage: this wave's own 16 * 128 words of LDS.
template <int K2, int CB>
__device__ __forceinline__ void wave_block(const uint16_t* xr, const uint32_t* tiles, int64_t stride_k, int pr0, int pr1,
                                           uint32_t* stage, int lane, int L, int h, f32x4_t (&acc)[8]) {
  constexpr int TW = tile_words<K2>();
  // The stored words of a k-tile pair (two runs of 8 tiles) come in with coalesced loads, a dword a lane, one pair
  // ahead, and go through the wave's own part of LDS: each lane then reads the two or three words its windows
  // start in.  (A lane loading its words itself costs sixteen times the load instructions, and the kernel was
  // bound by their issue.)  A staged tile repeats its first two words at its end, so a window never wraps.
  constexpr int NW = Windows<K2>::NW;
  constexpr int TWP = TW + 2, RUN = 8 * TW, GL = (RUN + 63) / 64;
  const Windows<K2> win(L, h);
  uint32_t g[2][GL];
  u32x4_t av, an;
  auto fetch = [&](int pr, uint32_t (&w)[2][GL], u32x4_t& a) {
    const uint32_t* xk = reinterpret_cast<const uint32_t*>(xr + 32 * pr);
    a = (u32x4_t){xk[0], xk[4], xk[8], xk[12]};
#pragma unroll
    for (int r = 0; r < 2; ++r) {
      const uint32_t* run = tiles + (size_t)(2 * pr + r) * stride_k;
#pragma unroll
      for (int i = 0; i < GL; ++i) w[r][i] = lane + 64 * i < RUN ? run[lane + 64 * i] : 0u;
    }
  };
  auto put = [&](const uint32_t (&w)[2][GL]) {
#pragma unroll
    for (int r = 0; r < 2; ++r)
#pragma unroll
      for (int i = 0; i < GL; ++i) {
        const int idx = lane + 64 * i, j = idx / TW, q = idx - j * TW;
        if (idx < RUN) {
          stage[(8 * r + j) * TWP + q] = w[r][i];
          if (q < 2) stage[(8 * r + j) * TWP + TW + q] = w[r][i];
        }
      }
  };
  if (pr0 < pr1) fetch(pr0, g, av);
  for (int pr = pr0; pr < pr1; ++pr) {
    put(g);
    __builtin_amdgcn_wave_barrier();         // the wave's LDS accesses run in program order: no wait beyond the data's
    fetch(pr + 1 < pr1 ? pr + 1 : pr, g, an);
    const f16x8_t a = __builtin_bit_cast(f16x8_t, av);
    // 3inst and mcg: a value is the sum of the two fp16 halves of its hashed word.  The matrix unit adds them: the
    // four hashed words of a tile are the B operand as they stand (eight fp16 numbers) against every input twice
    // over, so the add costs no vector instruction.  The products are exact in fp32, so each weight enters as the
    // exact sum of its halves (the stored value is that sum rounded to fp16: at most 2^-12 relative apart).
    f16x8_t a0, a1;
    if constexpr (CB != 2) {
      const u32x4_t lo = {__builtin_amdgcn_perm(av[0], av[0], 0x01000100u), __builtin_amdgcn_perm(av[0], av[0], 0x03020302u),
                          __builtin_amdgcn_perm(av[1], av[1], 0x01000100u), __builtin_amdgcn_perm(av[1], av[1], 0x03020302u)};
      const u32x4_t hi = {__builtin_amdgcn_perm(av[2], av[2], 0x01000100u), __builtin_amdgcn_perm(av[2], av[2], 0x03020302u),
                          __builtin_amdgcn_perm(av[3], av[3], 0x01000100u), __builtin_amdgcn_perm(av[3], av[3], 0x03020302u)};
      a0 = __builtin_bit_cast(f16x8_t, lo);
      a1 = __builtin_bit_cast(f16x8_t, hi);
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      uint32_t w0[NW], w1[NW];
#pragma unroll
      for (int q = 0; q < NW; ++q) {
        w0[q] = stage[j * TWP + win.wi + q];
        w1[q] = stage[(8 + j) * TWP + win.wi + q];
      }
      if constexpr (CB != 2) {
        uint32_t s0[4], s1[4];
        win.states(w0, s0);
        win.states(w1, s1);
        const u32x4_t x0 = {code_word<CB>(s0[0]), code_word<CB>(s0[1]), code_word<CB>(s0[2]), code_word<CB>(s0[3])};
        const u32x4_t x1 = {code_word<CB>(s1[0]), code_word<CB>(s1[1]), code_word<CB>(s1[2]), code_word<CB>(s1[3])};
        acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a0, __builtin_bit_cast(f16x8_t, x0), acc[j], 0, 0, 0);
        acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a1, __builtin_bit_cast(f16x8_t, x1), acc[j], 0, 0, 0);
      } else {
        uint32_t b0, b1, b2, b3;
        decode4<K2, CB>(win, w0, b0, b1);
        decode4<K2, CB>(win, w1, b2, b3);
        const u32x4_t bw = {b0, b1, b2, b3};
        const f16x8_t b = __builtin_bit_cast(f16x8_t, bw);
        acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, acc[j], 0, 0, 0);
      }
    }
    __builtin_amdgcn_wave_barrier();
    av = an;
  }
}

// every width ExLlamaV3 writes: k2 = 2 * bits; half-integer widths exist with the mul1 codebook only
#define TF_EXL3_WIDTHS(X, CB) X(2, CB) X(4, CB) X(6, CB) X(8, CB) X(10, CB) X(12, CB) X(14, CB) X(16, CB)
#define TF_EXL3_ALL(X) TF_EXL3_WIDTHS(X, 0) TF_EXL3_WIDTHS(X, 1) TF_EXL3_WIDTHS(X, 2) X(3, 2) X(5, 2) X(7, 2)
// every half-bit count from 2 to 16 with every codebook: what the routed experts and the plain decode accept
// (reference: cuda/exl3/experts.py:15-16, experts_grouped.cuh:184-187)
#define TF_EXL3_ODD(X, CB) X(3, CB) X(5, CB) X(7, CB) X(9, CB) X(11, CB) X(13, CB) X(15, CB)
#define TF_EXL3_EVERY(X) \
  TF_EXL3_WIDTHS(X, 0) TF_EXL3_ODD(X, 0) TF_EXL3_WIDTHS(X, 1) TF_EXL3_ODD(X, 1) TF_EXL3_WIDTHS(X, 2) TF_EXL3_ODD(X, 2)

}  // namespace
}  // namespace tf

#endif  // TF_EXL3_DECODE_H
