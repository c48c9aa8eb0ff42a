// Prefill-form 4-bit matmuls on the matrix cores: the token-sorted grouped expert GEMM (tf_experts_prefill) and the
// dense prompt matmul (tf_qmm_prefill).  Each weight is rounded once, K is one fp32 chain in order, so a row's bits
// depend neither on its item nor on its chunk (the contract of the reference's experts_prefill.cu:1, qmm_prefill.cu:1).
//
// Rounding.  The reference rounds the dequantized weight to bf16; against a dequant-then-matmul in fp32 that alone
// costs 2.4e-3 to 4.7e-3 relative L2 on the benchmark shapes, past the 2e-3 bound.  Here the weight is rounded to
// fp16 instead (11 significant bits): w16 = fp16(fma(q, 256 s, 256 b)), the activations go to fp16 exactly (a bf16
// value is an fp16 value unless it is below 2^-14, where it keeps 2^-24 absolute, or above 65504, where it is
// clamped), v_mfma_f32_16x16x32_f16 accumulates in fp32 and the sum is scaled back by 2^-8.  Same MFMA rate as
// bf16, an eighth of the rounding error, and the packed fp16 fma dequantizes two weights an instruction.
//
// A workgroup of four waves takes (item of up to 16*RT rows) x (128 columns); each wave owns 32 columns and all the
// item's rows.  The gathered activation rows are staged through LDS (64 inputs a step, double-buffered).  Lane
// (column c, quarter kq) of the MFMA's B operand needs the eight inputs 8 kq .. 8 kq + 7 of column c, which is
// exactly one packed word, and dequantizes it in registers; in the four-wave kernels each lane loads its own word,
// in the eight-wave ones a lane loads a column's four words at once and they change lanes by swaps.  A nibble in a byte is the e4m3 number q * 2^-9, so v_cvt_scalef32_pk_f16_fp8 with
// scale 2^9 turns two nibble-bytes into the fp16 pair (q0, q1); the operand order this gives, inputs
// (0, 4, 1, 5, 2, 6, 3, 7) of the eight, is applied to the activations when they are staged.

#include "tf_common.h"

namespace tf {
namespace {

constexpr int KSTEP = 64;                      // inputs staged a step
constexpr int AROW = KSTEP * 2 + 16;           // bytes of an LDS row: 128 of data, 16 of padding against conflicts

constexpr float WSCALE = 256.f, WUNSCALE = 1.f / 256.f;     // weights ride the MFMA scaled by 2^8 (see above)

typedef __attribute__((ext_vector_type(2))) _Float16 f16x2_t;

// eight consecutive bf16 inputs -> fp16 in the operand order (0, 4, 1, 5, 2, 6, 3, 7).  The conversion rounds toward
// zero, which is exact for every bf16 value in fp16's normal range and saturates a finite one beyond it at 65504.
__device__ __forceinline__ uint4 stage8(uint4 v) {
  const uint32_t d[4] = {v.x, v.y, v.z, v.w};
  float f[8];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    f[2 * i] = bf16_lo(d[i]);
    f[2 * i + 1] = bf16_hi(d[i]);
  }
  auto pk = [](float a, float b) { return __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(a, b)); };
  return make_uint4(pk(f[0], f[4]), pk(f[1], f[5]), pk(f[2], f[6]), pk(f[3], f[7]));
}

// A column's stored (scale | bias << 16) bf16 pair -> (fp16(256 s) | fp16(256 b) << 16).  Adding 8 to both exponents
// is the multiplication; bf16 -> fp16 is exact in fp16's normal range.
__device__ __forceinline__ uint32_t sb_half2(uint32_t v) {
  const uint32_t u = v + 0x04000400u;
  return __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(__uint_as_float(u << 16), __uint_as_float(u & 0xFFFF0000u)));
}

// The same from a scale and a bias still apart (each a bf16 in the low half of its register): the dense layout keeps
// them in two arrays, and joining them when they are loaded would make every step wait for loads it has just issued.
__device__ __forceinline__ uint32_t sb_half2(uint2 v) {
  return __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(__uint_as_float((v.x + 0x0400u) << 16),
                                                                  __uint_as_float((v.y + 0x0400u) << 16)));
}

// q * s + b on two fp16 lanes, s and b being the low and high half of one register (the splats fold into the
// packed instruction's operand selects)
__device__ __forceinline__ f16x2_t fma_sb(f16x2_t q, uint32_t sb) {
  const f16x2_t v = __builtin_bit_cast(f16x2_t, sb);
  return __builtin_elementwise_fma(q, __builtin_shufflevector(v, v, 0, 0), __builtin_shufflevector(v, v, 1, 1));
}

// one packed word -> the B operand, inputs in the order (0, 4, 1, 5, 2, 6, 3, 7), each fp16(fma(q, 256 s, 256 b))
__device__ __forceinline__ f16x8_t dequant8h(uint32_t w, uint32_t sb) {
  const uint32_t lo = w & 0x0F0F0F0Fu, hi = (w >> 4) & 0x0F0F0F0Fu;
  const f16x2_t w0 = fma_sb(__builtin_amdgcn_cvt_scalef32_pk_f16_fp8(lo, 512.f, false), sb);
  const f16x2_t w1 = fma_sb(__builtin_amdgcn_cvt_scalef32_pk_f16_fp8(lo, 512.f, true), sb);
  const f16x2_t w2 = fma_sb(__builtin_amdgcn_cvt_scalef32_pk_f16_fp8(hi, 512.f, false), sb);
  const f16x2_t w3 = fma_sb(__builtin_amdgcn_cvt_scalef32_pk_f16_fp8(hi, 512.f, true), sb);
  f16x8_t r;
  r[0] = w0[0]; r[1] = w0[1]; r[2] = w1[0]; r[3] = w1[1];
  r[4] = w2[0]; r[5] = w2[1]; r[6] = w3[0]; r[7] = w3[1];
  return r;
}

// ---- the reference's own prompt arithmetic (AR = 1): bf16 operands, w = bf16(fma(q, s, b)) ------------------------------
//
// cuda/kernels/qmm_prefill.cu:116-117 and cuda/experts_prefill.cu:130-131 round every dequantized weight to bf16 and
// run a bf16 mma.  That form has bf16's range on both operands (no clamp at 65504, any scale or bias), at twice the
// dequantization work and eight times the rounding error of the fp16 form above; it is what callers get when a
// table's scales or biases do not fit fp16 after the 2^8 scaling, or when they ask for it.

// eight consecutive bf16 inputs in the operand order (0, 4, 1, 5, 2, 6, 3, 7), unchanged
__device__ __forceinline__ uint4 stage8_bf16(uint4 v) {
  return make_uint4(__builtin_amdgcn_perm(v.z, v.x, 0x05040100u), __builtin_amdgcn_perm(v.z, v.x, 0x07060302u),
                    __builtin_amdgcn_perm(v.w, v.y, 0x05040100u), __builtin_amdgcn_perm(v.w, v.y, 0x07060302u));
}

__device__ __forceinline__ uint32_t pack_bf16_rn(float lo, float hi) {
  typedef __attribute__((ext_vector_type(2))) __bf16 bf2;
  bf2 r;
  r[0] = (__bf16)lo;
  r[1] = (__bf16)hi;
  return __builtin_bit_cast(uint32_t, r);
}

// one packed word -> the B operand in the same input order, each bf16(fma(q, s, b)) with s and b the stored bf16
// values: round to nearest even, as the reference's __float2bfloat16_rn
__device__ __forceinline__ bf16x8_t dequant8b(uint32_t w, uint32_t sb) {
  const float s = bf16_lo(sb), b = bf16_hi(sb);
  uint32_t lo = w & 0x0F0F0F0Fu, hi = (w >> 4) & 0x0F0F0F0Fu;
  // the compiler is not to know that these are w's nibbles: knowing it, it extracts each of the eight from w and
  // converts that (16 instructions), where a byte of lo or hi converts as it lies (v_cvt_f32_ubyte0..3: 8)
  asm("" : "+v"(lo));
  asm("" : "+v"(hi));
  auto q = [](uint32_t v, int byte) { return (float)((v >> (8 * byte)) & 0xFFu); };
  const u32x4_t r = {pack_bf16_rn(fmaf(q(lo, 0), s, b), fmaf(q(lo, 1), s, b)),
                     pack_bf16_rn(fmaf(q(lo, 2), s, b), fmaf(q(lo, 3), s, b)),
                     pack_bf16_rn(fmaf(q(hi, 0), s, b), fmaf(q(hi, 1), s, b)),
                     pack_bf16_rn(fmaf(q(hi, 2), s, b), fmaf(q(hi, 3), s, b))};
  return __builtin_bit_cast(bf16x8_t, r);
}

// EPI 0: fp32; 1: bf16 relu(bf16 a)^2; 2: bf16 SwiGLU(matrix 0, matrix 1); 3: bf16; 4: fp16, values beyond its
// range stored as +-65504 (pair outputs at half the bytes of fp32 and an eighth of bf16's rounding)
template <int EPI>
__device__ __forceinline__ void store_out(void* out, size_t at, float a, float u, float limit) {
  if constexpr (EPI == 0) reinterpret_cast<float*>(out)[at] = a;
  else if constexpr (EPI == 1) reinterpret_cast<uint16_t*>(out)[at] = (uint16_t)f32_bf16_bits(relu2(a));
  else if constexpr (EPI == 2) reinterpret_cast<uint16_t*>(out)[at] = (uint16_t)f32_bf16_bits(swiglu(a, u, limit));
  else if constexpr (EPI == 4) reinterpret_cast<_Float16*>(out)[at] = (_Float16)fminf(fmaxf(a, -65504.f), 65504.f);
  else reinterpret_cast<uint16_t*>(out)[at] = (uint16_t)f32_bf16_bits(a);
}

// Which way round a tile comes out of the matrix instruction.  Activations first: D[row 4 kq + i][column c], a lane
// holds one column of four rows.  Weights first (SWAP): D[column 4 kq + i][row c], a lane holds four consecutive
// columns of one row, which leave as one 8- or 16-byte store (or, STAGE_OUT, go to LDS as one write so that whole
// rows leave side by side).  The products and their order along K are the same, and so are the bits (the kernels
// of one family are tested equal across the forms).  Which form is faster is a matter of what the compiler makes of
// the loop around it, so it is a parameter of the body and each instance takes what it measured best with, side by
// side on one box: the dense prompt matmul SWAP (4096 cubed: 177 -> 141 us with the bf16 arithmetic, 144 -> 143 with
// the fp16 one), the experts' down projection SWAP with STAGE_OUT (config 3: 232 -> 222 us), the experts' gate and up
// neither (342 -> 350 us with them).

// Four consecutive columns of one row (a SWAP lane's share of a tile): one store where the row's length allows
// (n a multiple of 4: the columns are whole and aligned), else element by element.  `at`: index of the first of the
// four; `left`: columns from it to the row's end.
template <int EPI>
__device__ __forceinline__ void store4(void* out, size_t at, const float (&a)[4], const float (&u)[4], float limit,
                                       int left, bool whole) {
  if (left <= 0) return;
  if (!whole) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (i < left) store_out<EPI>(out, at + i, a[i], u[i], limit);
    return;
  }
  if constexpr (EPI == 0) {
    *reinterpret_cast<float4*>(reinterpret_cast<float*>(out) + at) = make_float4(a[0], a[1], a[2], a[3]);
  } else if constexpr (EPI == 4) {
    auto h = [](float lo, float hi) {
      const _Float16 l = (_Float16)fminf(fmaxf(lo, -65504.f), 65504.f), g = (_Float16)fminf(fmaxf(hi, -65504.f), 65504.f);
      return (uint32_t)__builtin_bit_cast(uint16_t, l) | ((uint32_t)__builtin_bit_cast(uint16_t, g) << 16);
    };
    *reinterpret_cast<uint2*>(reinterpret_cast<uint16_t*>(out) + at) = make_uint2(h(a[0], a[1]), h(a[2], a[3]));
  } else {
    float v[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = EPI == 1 ? relu2(a[i]) : EPI == 2 ? swiglu(a[i], u[i], limit) : a[i];
    *reinterpret_cast<uint2*>(reinterpret_cast<uint16_t*>(out) + at) = make_uint2(pack_bf16(v[0], v[1]), pack_bf16(v[2], v[3]));
  }
}

// The shared body.  SRC gives, for the workgroup's item: rows(), src_row(r), dst_row(r); WSRC gives the lane's
// packed word and its column's scale and bias.
//   word(g, m, i, t): group g, matrix m, chunk i (32 inputs) of the group, column tile t (16 columns) of the wave
//   sb(g, m, t): that column's stored (scale | bias << 16) pair of group g
template <int GS, int NM, int EPI, int RT, int AR, bool SWAP, class WSRC>
__device__ __forceinline__ void mfma_body(const uint16_t* __restrict__ X, int64_t x_stride, int K, const WSRC& ws,
                                          const int* src_rows, int cnt, void* out, int N, int col0, int wave_cols_ok,
                                          const int* dst_rows, float limit, unsigned char* smem) {
  constexpr int ROWS = 16 * RT;
  constexpr int CPS = KSTEP / 32;              // chunks a step
  constexpr int GPS = KSTEP / GS;              // groups a step (1 or 2)
  constexpr int PIECES = ROWS * 8;             // 16-byte pieces of a staged tile
  constexpr int PPT = (PIECES + 255) / 256;
  const int tid = threadIdx.x, lane = tid & 63, c = lane & 15, kq = lane >> 4;
  const int steps = (K + KSTEP - 1) / KSTEP;

  // this thread's pieces of the activation tile
  const uint16_t* asrc[PPT];
  int adst[PPT];
#pragma unroll
  for (int j = 0; j < PPT; ++j) {
    const int q = tid + j * 256, r = q >> 3, ch = q & 7;
    adst[j] = -1;
    asrc[j] = X;
    if (q < PIECES) {
      adst[j] = r * AROW + ch * 16;
      asrc[j] = X + (size_t)src_rows[r < cnt ? r : cnt - 1] * x_stride + ch * 8;
    }
  }
  auto load_a = [&](int step, uint4 (&v)[PPT]) {
#pragma unroll
    for (int j = 0; j < PPT; ++j) {
      const int q = tid + j * 256, ch = q & 7;
      v[j] = make_uint4(0u, 0u, 0u, 0u);
      if (adst[j] >= 0 && step * KSTEP + ch * 8 < K) v[j] = *reinterpret_cast<const uint4*>(asrc[j] + (size_t)step * KSTEP);
    }
  };
  auto store_a = [&](int buf, const uint4 (&v)[PPT]) {
#pragma unroll
    for (int j = 0; j < PPT; ++j)
      if (adst[j] >= 0)
        *reinterpret_cast<uint4*>(smem + buf * (ROWS * AROW) + adst[j]) = AR ? stage8_bf16(v[j]) : stage8(v[j]);
  };

  uint32_t wcur[NM][CPS][2], wnxt[NM][CPS][2];
  uint32_t scur[NM][GPS][2], snxt[NM][GPS][2];
  auto load_w = [&](int step, uint32_t (&w)[NM][CPS][2], uint32_t (&s)[NM][GPS][2]) {
#pragma unroll
    for (int m = 0; m < NM; ++m)
#pragma unroll
      for (int t = 0; t < 2; ++t) {
#pragma unroll
        for (int i = 0; i < CPS; ++i) {
          const int k0 = step * KSTEP + 32 * i;
          w[m][i][t] = k0 < K ? ws.word(k0 / GS, m, (k0 % GS) / 32, t) : 0u;
        }
#pragma unroll
        for (int gi = 0; gi < GPS; ++gi) {
          const int k0 = step * KSTEP + GS * gi;
          s[m][gi][t] = k0 < K ? ws.sb(k0 / GS, m, t) : 0u;
        }
      }
  };

  f32x4_t acc[NM][RT][2];
#pragma unroll
  for (int m = 0; m < NM; ++m)
#pragma unroll
    for (int r = 0; r < RT; ++r)
#pragma unroll
      for (int t = 0; t < 2; ++t) acc[m][r][t] = (f32x4_t){0.f, 0.f, 0.f, 0.f};

  const int nt = (cnt + 15) >> 4;              // row tiles in use
  uint4 areg[PPT];
  load_a(0, areg);
  load_w(0, wcur, scur);
  store_a(0, areg);
  __syncthreads();
  for (int step = 0; step < steps; ++step) {
    const bool more = step + 1 < steps;
    if (more) {
      load_a(step + 1, areg);
      load_w(step + 1, wnxt, snxt);
    }
    const unsigned char* abuf = smem + (step & 1) * (ROWS * AROW);
#pragma unroll
    for (int i = 0; i < CPS; ++i) {
      if (step * KSTEP + 32 * i >= K) break;
      u32x4_t bfrag[NM][2];
#pragma unroll
      for (int m = 0; m < NM; ++m)
#pragma unroll
        for (int t = 0; t < 2; ++t) {
          const int gi = (32 * i) / GS;
          if constexpr (AR) bfrag[m][t] = __builtin_bit_cast(u32x4_t, dequant8b(wcur[m][i][t], scur[m][gi][t]));
          else bfrag[m][t] = __builtin_bit_cast(u32x4_t, dequant8h(wcur[m][i][t], sb_half2(scur[m][gi][t])));
        }
#pragma unroll
      for (int r = 0; r < RT; ++r) {
        if (r >= nt) break;
        const u32x4_t a = *reinterpret_cast<const u32x4_t*>(abuf + (16 * r + c) * AROW + i * 64 + kq * 16);
#pragma unroll
        for (int m = 0; m < NM; ++m)
#pragma unroll
          for (int t = 0; t < 2; ++t) {
            const u32x4_t first = SWAP ? bfrag[m][t] : a, second = SWAP ? a : bfrag[m][t];
            if constexpr (AR)
              acc[m][r][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                  __builtin_bit_cast(bf16x8_t, first), __builtin_bit_cast(bf16x8_t, second), acc[m][r][t], 0, 0, 0);
            else
              acc[m][r][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(
                  __builtin_bit_cast(f16x8_t, first), __builtin_bit_cast(f16x8_t, second), acc[m][r][t], 0, 0, 0);
          }
      }
    }
    if (more) {
      store_a((step + 1) & 1, areg);
#pragma unroll
      for (int m = 0; m < NM; ++m) {
#pragma unroll
        for (int i = 0; i < CPS; ++i)
#pragma unroll
          for (int t = 0; t < 2; ++t) wcur[m][i][t] = wnxt[m][i][t];
#pragma unroll
        for (int gi = 0; gi < GPS; ++gi)
#pragma unroll
          for (int t = 0; t < 2; ++t) scur[m][gi][t] = snxt[m][gi][t];
      }
    }
    __syncthreads();
  }
  if (!wave_cols_ok) return;
  if constexpr (SWAP) {
    // a lane holds row 16 r + c, columns 16 t + 4 kq + (0..3) of each 16 x 16 tile
    const bool whole = N % 4 == 0;
#pragma unroll
    for (int r = 0; r < RT; ++r) {
      if (r >= nt) break;
      const int row = 16 * r + c;
      if (row >= cnt) continue;
      const size_t base = (size_t)dst_rows[row] * N;
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        const int col = col0 + 16 * t + 4 * kq;
        float a4[4], u4[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          a4[i] = acc[0][r][t][i] * (AR ? 1.f : WUNSCALE);
          u4[i] = acc[NM - 1][r][t][i] * (AR ? 1.f : WUNSCALE);
        }
        store4<EPI>(out, base + col, a4, u4, limit, N - col, whole);
      }
    }
    return;
  }
  // D[row 4 kq + i][column c] of each 16 x 16 tile
#pragma unroll
  for (int r = 0; r < RT; ++r) {
    if (r >= nt) break;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int row = 16 * r + 4 * kq + i;
      if (row >= cnt) continue;
      const size_t base = (size_t)dst_rows[row] * N;
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        const int col = col0 + 16 * t + c;
        if (col < N)
          store_out<EPI>(out, base + col, acc[0][r][t][i] * (AR ? 1.f : WUNSCALE),
                         acc[NM - 1][r][t][i] * (AR ? 1.f : WUNSCALE), limit);
      }
    }
  }
}

// ---- routed experts ----------------------------------------------------------------------------------------------------

template <int GS, int NM>
struct ExpertWords {
  const uint32_t* base;      // the lane's (expert, column block): + c * 4 + kq applied
  const uint32_t* sbase;
  __device__ __forceinline__ uint32_t word(int g, int m, int i, int t) const {
    return base[((size_t)g * NM + m) * block_words(GS) + i * 128 + t * 64];
  }
  __device__ __forceinline__ uint32_t sb(int g, int m, int t) const {
    return sbase[((size_t)g * NM + m) * block_words(GS) + t * 16];
  }
};

template <int GS, int NM, int EPI, int RT, int AR>
__global__ void __launch_bounds__(256)
    experts_prefill_kernel(const uint16_t* __restrict__ X, int64_t x_stride, int slots, const uint32_t* __restrict__ W,
                           int KG, int NB, const int* __restrict__ items, const int* __restrict__ counts,
                           const int* __restrict__ members, void* __restrict__ out, int N, float limit) {
  extern __shared__ __align__(16) unsigned char smem[];
  __shared__ int src_rows[16 * RT], dst_rows[16 * RT];
  const int nbt = (NB + 3) >> 2;
  const int it = blockIdx.x / nbt, cbt = blockIdx.x - it * nbt;
  if (it >= counts[0]) return;
  const int e = items[3 * it], first = items[3 * it + 1], cnt = min(items[3 * it + 2], 16 * RT);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, c = lane & 15, kq = lane >> 4;
  if (tid < 16 * RT) {
    const int p = members[first + (tid < cnt ? tid : 0)];
    dst_rows[tid] = p;
    src_rows[tid] = slots ? p / slots : p;
  }
  __syncthreads();
  const int nb = cbt * 4 + wave;
  const bool ok = nb < NB;
  ExpertWords<GS, NM> ws;
  const uint32_t* blk = W + (((size_t)e * NB + (ok ? nb : NB - 1)) * KG) * (size_t)(NM * block_words(GS));
  ws.base = blk + c * 4 + kq;
  ws.sbase = blk + 32 * GS / 8 + c;
  mfma_body<GS, NM, EPI, RT, AR, false>(X, x_stride, KG * GS, ws, src_rows, cnt, out, N, nb * 32, ok, dst_rows, limit, smem);
}

// ---- routed experts, big items ---------------------------------------------------------------------------------------
//
// An item of up to 128 pairs against 512 weight columns (NM = 1: 512 output columns; NM = 2: 256 output columns of
// gate and of up).  Each of the eight waves owns 64 weight columns = four B operands and all eight 16-row tiles, so
// one dequantized operand feeds eight MFMAs and one LDS read of the activations feeds four: per 32 inputs a wave
// issues 32 MFMAs against 8 LDS reads and 4 dequantizations.  Weights are requested a step and a half (96 inputs)
// ahead into registers and change lanes there, activations one step ahead through registers into the workgroup's
// two LDS stages, one barrier a step.  The arithmetic of a row (operand values, MFMA, K order) is the small kernel's, so the bits are too.

constexpr int BIG_ROWS = 128;
constexpr int BIG_WAVES = 8;
constexpr int BIG_THREADS = BIG_WAVES * 64;
// LDS of a workgroup: two stages of activations
constexpr int BIG_LDS = 2 * BIG_ROWS * AROW;
static_assert(BIG_LDS + 2 * 2 * BIG_ROWS * 4 + 16 <= 64 * 1024, "within what a launch gets without asking");

// The pipeline for an item of at most 16 * RT rows (RT = 2, 4 or 8).  K is a multiple of KSTEP and nothing inside a
// step is conditional (prefetches past the end re-read the last step, rows past the item read its first row), so the
// compiler is free to keep the LDS reads of the next row tile in flight under the MFMAs of this one.
// Where a wave's weights come from.  A wave takes 64 weight columns (four operands of 16), and for loading them lane L
// owns column L: load(step, raw) requests the column's four packed words of each 32-input chunk of the step as ONE
// 16-byte load (both layouts keep a column's four words of 32 inputs side by side) and its scale and bias of each
// group of the step, i.e. 4 to 6 load instructions a wave and step where a word a lane and operand took 16.  (A
// wave's load instruction keeps the compute unit's address unit busy for about 16 cycles whatever its width: with a
// word a lane the short items, which mostly stream their tables, ran at 3 TB/s with that unit busy 60 % of the time.)
// The lane that multiplies is another one (lane (c, kq) takes words kq of columns 16 j + c), so the words change
// lanes on their way: by the chip's lane-swap instructions, in registers (big_body's `across`).
// Buffer loads: the base in scalar registers, the step as the scalar offset, the lane's part as the vector offset and
// the chunk or group as the immediate, so no address arithmetic is left on the vector unit.
template <int GS, int NM>
struct ExpertSource {
  static constexpr int CPS = KSTEP / 32, GPS = KSTEP / GS;
  static constexpr bool KEEPS_GROUP_WORDS = false;
  static constexpr uint32_t GSTRIDE = NM * block_words(GS);      // words from one group to the next
  struct Raw {
    u32x4_t q[CPS];
    uint32_t sb[GPS];
  };
  __amdgpu_buffer_rsrc_t rsrc;                                    // one expert's matrices
  uint32_t qp, sp;      // byte offsets inside the expert (below 2^32): the column's words of group 0; its (scale | bias << 16)
  __device__ __forceinline__ void load(int step, Raw& r) const {
    const int soff = step * (int)(GPS * GSTRIDE * 4);
#pragma unroll
    for (int i = 0; i < CPS; ++i)
      r.q[i] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, qp + (((32 * i) / GS) * GSTRIDE + (((32 * i) % GS) / 32) * 128) * 4,
                                                     soff, 0);
#pragma unroll
    for (int gi = 0; gi < GPS; ++gi) r.sb[gi] = __builtin_amdgcn_raw_buffer_load_b32(rsrc, sp + gi * GSTRIDE * 4, soff, 0);
  }
  // the column's stored (scale | bias << 16) of group gi of the step
  static __device__ __forceinline__ uint32_t sb_word(const Raw& r, int gi) { return r.sb[gi]; }
};

// The dense layout: codes [n / 64][K / gs][gs / 32][64][4] words, scales and biases bf16 [K / gs][npad].
template <int GS>
struct DenseSource {
  static constexpr int CPS = KSTEP / 32, GPS = KSTEP / GS;
  static constexpr bool KEEPS_GROUP_WORDS = true;
  struct Raw {
    u32x4_t q[CPS];
    uint32_t s[GPS], b[GPS];          // each a bf16 in the low half, joined when a chunk is taken (not when they
  };                                  // are requested: that would wait for loads just issued)
  __amdgpu_buffer_rsrc_t codes, scales, biases;
  uint32_t qp, cp;                                                // byte offsets: the column's four words; its bf16
  int row_bytes;                                                  // bytes from one group's scales to the next
  __device__ __forceinline__ void load(int step, Raw& r) const {
    const int soff = step * (KSTEP / 32) * 1024;                  // 32 inputs of a 64-column tile are 1 KB of codes
#pragma unroll
    for (int i = 0; i < CPS; ++i) r.q[i] = __builtin_amdgcn_raw_buffer_load_b128(codes, qp + i * 1024, soff, 0);
#pragma unroll
    for (int gi = 0; gi < GPS; ++gi) {
      const int goff = (step * GPS + gi) * row_bytes;
      r.s[gi] = __builtin_amdgcn_raw_buffer_load_b16(scales, cp, goff, 0);
      r.b[gi] = __builtin_amdgcn_raw_buffer_load_b16(biases, cp, goff, 0);
    }
  }
  static __device__ __forceinline__ uint32_t sb_word(const Raw& r, int gi) { return (r.s[gi] & 0xFFFFu) | (r.b[gi] << 16); }
};

// AR: TF_ARITH_F16 (fp16 operands, weights scaled by 2^8) or TF_ARITH_BF16 (the reference's bf16(fma(q, s, b)) weights
// and untouched bf16 activations on the bf16 matrix instruction): the operand bits of mfma_body's two forms.
struct NoStaged {
  __device__ __forceinline__ void operator()() const {}
};

// `staged()` runs in every thread right after the barrier that ends the prologue: the first operands have arrived by
// then, and with them (a wave's vector memory operations complete in issue order) whatever the caller requested
// before calling, which it can put away there without a wait of its own.
template <int GS, int NM, int EPI, int RT, int AR, bool SWAP, class WS, int TJ = 4, int NTHREADS = BIG_THREADS,
          bool STAGE_OUT = false, class STAGED = NoStaged>
__device__ __forceinline__ void big_body(const uint16_t* __restrict__ X, int64_t x_stride, const WS& ws,
                                         const int (&ocol)[TJ], const bool (&jok)[TJ],
                                         int K, const int* src_rows, const int* dst_rows, int cnt,
                                         void* __restrict__ out, int N, float limit, unsigned char* smem,
                                         STAGED&& staged = STAGED(), int thread = -1) {
  constexpr int CPS = KSTEP / 32, GPS = KSTEP / GS;
  constexpr int ROWS = 16 * RT;
  constexpr int PIECES = ROWS * 8;                // 16-byte pieces of a staged tile
  constexpr int PPT = (PIECES + NTHREADS - 1) / NTHREADS;
  constexpr int STAGE = BIG_ROWS * AROW;
  const int tid = thread < 0 ? (int)threadIdx.x : thread, lane = tid & 63, c = lane & 15, kq = lane >> 4;
  const int steps = K / KSTEP;
  typedef typename WS::Raw Raw;
  static_assert(TJ == 4, "a wave takes 64 weight columns: four operands of 16");
  bool tile_ok[TJ];          // the lane's tile j exists at all (lane 0 of the tile's row of 16 says)
#pragma unroll
  for (int j = 0; j < TJ; ++j) tile_ok[j] = SWAP ? __shfl(jok[j] ? 1 : 0, lane & 48) != 0 : jok[j];
  // Lane L loads column L's four packed words of a chunk as one 16-byte load (a load instruction costs the address
  // unit the same 16 cycles whatever its width); the matrix instruction wants lane (column c, quarter kq) to hold
  // word kq of columns c, 16 + c, 32 + c, 48 + c.  That is the transpose of a 4 x 4 matrix whose rows are the wave's
  // four rows of 16 lanes and whose columns are the four registers, which this chip's two swap instructions do in
  // four steps (rows 2, 3 of one register against rows 0, 1 of another, then odd rows against even ones).  Four
  // copies of the column's scale and bias word transposed the same way are the four columns' words in every row;
  // for the fp16 form the word is made the fp16 pair first, once a column and group instead of once an operand.
  // With groups of 64 a step's two chunks share their scale and bias words; the dense kernel keeps them across the two
  // (2 % of its time).  The experts' kernels, a few registers fuller, would spill for it and transpose them again.
  constexpr bool KEEP_SB = WS::KEEPS_GROUP_WORDS && GS == 64;
  auto across = [](uint32_t (&v)[TJ]) {
    auto swap32 = [](uint32_t& x, uint32_t& y) {
      const auto r = __builtin_amdgcn_permlane32_swap(x, y, false, false);
      x = r[0], y = r[1];
    };
    auto swap16 = [](uint32_t& x, uint32_t& y) {
      const auto r = __builtin_amdgcn_permlane16_swap(x, y, false, false);
      x = r[0], y = r[1];
    };
    swap32(v[0], v[2]);
    swap32(v[1], v[3]);
    swap16(v[0], v[1]);
    swap16(v[2], v[3]);
  };
  auto take = [&](const Raw& r, int i, uint32_t (&w)[TJ], uint32_t (&sb)[TJ]) {
#pragma unroll
    for (int j = 0; j < TJ; ++j) w[j] = r.q[i][j];
    across(w);
    if (KEEP_SB && i % 2 == 1) return;          // the group of the chunk before: its columns' words are in sb still
    const uint32_t word = WS::sb_word(r, (32 * i) / GS);
    const uint32_t mine = AR ? word : sb_half2(word);
#pragma unroll
    for (int j = 0; j < TJ; ++j) sb[j] = mine;
    across(sb);
  };
  // this thread's pieces of the activation tile: piece q = (row q / 8, 16 bytes q % 8)
  const uint16_t* asrc[PPT];
#pragma unroll
  for (int j = 0; j < PPT; ++j) {
    const int q = tid + j * NTHREADS, r = q >> 3, ch = q & 7;
    asrc[j] = X + (size_t)src_rows[r < cnt ? r : 0] * x_stride + ch * 8;
  }
  auto load_a = [&](int step, uint4 (&v)[PPT]) {
#pragma unroll
    for (int j = 0; j < PPT; ++j)
      if (PIECES % NTHREADS == 0 || tid + j * NTHREADS < PIECES)
        v[j] = *reinterpret_cast<const uint4*>(asrc[j] + (size_t)step * KSTEP);
  };
  auto store_a = [&](int buf, const uint4 (&v)[PPT]) {
#pragma unroll
    for (int j = 0; j < PPT; ++j) {
      const int q = tid + j * NTHREADS;
      if (PIECES % NTHREADS == 0 || q < PIECES)
        *reinterpret_cast<uint4*>(smem + buf * STAGE + (q >> 3) * AROW + (q & 7) * 16) =
            AR ? stage8_bf16(v[j]) : stage8(v[j]);
    }
  };
  // one packed word and its column's scale and bias -> the B operand's eight values, as bits
  auto dequant = [](uint32_t w, uint32_t sb) {
    if constexpr (AR) return __builtin_bit_cast(u32x4_t, dequant8b(w, sb));
    else return __builtin_bit_cast(u32x4_t, dequant8h(w, sb));
  };
  auto mfma = [](u32x4_t a, u32x4_t b, f32x4_t c) {
    const u32x4_t first = SWAP ? b : a, second = SWAP ? a : b;
    if constexpr (AR)
      return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, first), __builtin_bit_cast(bf16x8_t, second), c, 0, 0, 0);
    else
      return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8_t, first), __builtin_bit_cast(f16x8_t, second), c, 0, 0, 0);
  };
  constexpr float UNSCALE = AR ? 1.f : WUNSCALE;

  f32x4_t acc[TJ][RT];
#pragma unroll
  for (int j = 0; j < TJ; ++j)
#pragma unroll
    for (int r = 0; r < RT; ++r) acc[j][r] = (f32x4_t){0.f, 0.f, 0.f, 0.f};

  // Two landing sets of registers: step t's words are requested into set t & 1 in the middle of step t - 2, a moment
  // after that set's last chunk has been taken, and are taken a chunk ahead of their MFMAs (the first in the last
  // chunk of step t - 1).
  static_assert(CPS == 2, "a step is two chunks: the landing set is free after the first");
  Raw raw[2];
  uint4 ar[PPT];
  const int last = steps - 1;
  ws.load(0, raw[0]);
  load_a(0, ar);
  ws.load(min(1, last), raw[1]);
  store_a(0, ar);
  // Software pipeline: the operands of the NEXT 32 inputs are dequantized under the MFMAs of these 32 (chunk i's are
  // bb[i], and it makes bb[1 - i]).  And a step's last row tile waits until the barrier is behind: its four MFMAs run
  // at the head of the next step, while that step's first activation operands are on their way from LDS (before
  // the first step they multiply zeros).
  u32x4_t bb[2][TJ], alast = {0u, 0u, 0u, 0u};
  uint32_t sn_step[TJ];          // KEEP_SB: the four columns' scale and bias words of the group last taken
  {
    uint32_t wn[TJ];
    uint32_t (&sn)[TJ] = sn_step;
    take(raw[0], 0, wn, sn);
#pragma unroll
    for (int j = 0; j < TJ; ++j) {
      bb[0][j] = dequant(wn[j], sn[j]);
      bb[1][j] = (u32x4_t){0u, 0u, 0u, 0u};
    }
  }
  constexpr bool DEFER = RT == 8;          // with fewer row tiles a step the tile put off is too large a part of it
  auto last_tile = [&]() {
    if constexpr (!DEFER) return;
#pragma unroll
    for (int j = 0; j < TJ; ++j) acc[j][RT - 1] = mfma(alast, bb[1][j], acc[j][RT - 1]);
  };
  __syncthreads();
  staged();
  TF_MARK(2);
  for (int step0 = 0; step0 < steps; step0 += 2) {
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int step = step0 + u;
      if (step < steps) {
        // stage `u` of LDS holds this step's activations; the next step's are requested now and staged at the end
        // of the step
        load_a(min(step + 1, last), ar);
        const unsigned char* abuf = smem + u * STAGE + c * AROW + kq * 16;
        // activation operands are requested two row tiles before their MFMAs (an LDS read takes about as long as
        // one row tile's four MFMAs): operand t of the step is (chunk t / RT, row tile t % RT)
        auto read_a = [&](int t) {
          return *reinterpret_cast<const u32x4_t*>(abuf + 16 * (t % RT) * AROW + (t / RT) * 64);
        };
        u32x4_t a = read_a(0), a1 = read_a(1);
        last_tile();
#pragma unroll
        for (int i = 0; i < CPS; ++i) {
          uint32_t wn[TJ], sn_chunk[TJ];
          uint32_t (&sn)[TJ] = KEEP_SB ? sn_step : sn_chunk;                      // the next chunk's words: this step's, or the next step's first
          if (i + 1 < CPS) take(raw[u], i + 1, wn, sn);
          else take(raw[1 - u], 0, wn, sn);
#pragma unroll
          for (int r = 0; r < RT; ++r) {
            const int t = i * RT + r;
            u32x4_t a2 = a1;
            if (t + 2 < CPS * RT) a2 = read_a(t + 2);
            if (DEFER && t == CPS * RT - 1) {
              alast = a;
            } else {
#pragma unroll
              for (int j = 0; j < TJ; ++j)
                acc[j][r] = mfma(a, bb[i][j], acc[j][r]);
            }
            a = a1;
            a1 = a2;
            // a share of the next chunk's dequantization rides along with each row tile
            constexpr int JPR = (TJ + RT - 1) / RT;          // operands a row tile (2, 1, 1 for RT = 2, 4, 8)
#pragma unroll
            for (int jj = 0; jj < JPR; ++jj) {
              const int j = r * JPR + jj;
              if (j < TJ) bb[1 - i][j] = dequant(wn[j], sn[j]);
            }
          }
          // this step's last words have been taken: their landing set takes the request for the step after next
          if (i == CPS - 2) ws.load(min(step + 2, last), raw[u]);
        }
        store_a(1 - u, ar);
        __syncthreads();
      }
    }
  }
  last_tile();
  TF_MARK(3);
  if constexpr (SWAP) {
    if (N % 32 == 0 && STAGE_OUT) {
      // Whole lines out: a lane's four columns of each tile go to the wave's own corner of LDS (free now: the loop
      // ended on a barrier) as one 8- or 16-byte write, and a row tile leaves as 16-byte pieces, a row's 32 or 64
      // columns side by side.  What the element-wise stores cost is the lines they touch (64 a row tile and wave, 32
      // bytes of each; a wave's stores take about 19 cycles a line): this way it is 8 or 16.
      constexpr int ES = EPI == 0 ? 4 : 2;                       // bytes an element
      constexpr int OJ = NM == 2 ? TJ / 2 : TJ;                  // 16-column tiles of output a wave
      constexpr int OROW = 16 * OJ * ES + 16;                    // bytes of a staged row (padded against bank conflicts)
      constexpr int CPR = 16 * OJ * ES / 16;                     // 16-byte pieces a row
      static_assert(BIG_WAVES * 16 * OROW <= 2 * STAGE, "the output tiles of a workgroup's waves fit the activation stages");
      unsigned char* mine = smem + (tid >> 6) * (16 * OROW);
      const int col0 = ocol[0] - c;                              // the wave's first output column (its tiles are neighbours)
      unsigned okmask = 0;
#pragma unroll
      for (int j = 0; j < OJ; ++j) okmask |= (tile_ok[j] ? 1u : 0u) << j;
      unsigned char* obytes = reinterpret_cast<unsigned char*>(out);
#pragma unroll
      for (int r = 0; r < RT; ++r) {
        if (16 * r >= cnt) break;
#pragma unroll
        for (int j = 0; j < OJ; ++j) {
          unsigned char* at = mine + c * OROW + (16 * j + 4 * kq) * ES;
          float v[4];
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const float a = acc[j][r][i] * UNSCALE, u = NM == 2 ? acc[j + TJ / 2][r][i] * UNSCALE : 0.f;
            v[i] = EPI == 1 ? relu2(a) : EPI == 2 ? swiglu(a, u, limit) : EPI == 4 ? fminf(fmaxf(a, -65504.f), 65504.f) : a;
          }
          if constexpr (EPI == 0) {
            *reinterpret_cast<float4*>(at) = make_float4(v[0], v[1], v[2], v[3]);
          } else if constexpr (EPI == 4) {
            auto h = [](float lo, float hi) {
              return (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)lo) | ((uint32_t)__builtin_bit_cast(uint16_t, (_Float16)hi) << 16);
            };
            *reinterpret_cast<uint2*>(at) = make_uint2(h(v[0], v[1]), h(v[2], v[3]));
          } else {
            *reinterpret_cast<uint2*>(at) = make_uint2(pack_bf16(v[0], v[1]), pack_bf16(v[2], v[3]));
          }
        }
        // a wave's LDS operations run in the order it issued them: the reads below see the writes above
#pragma unroll
        for (int q0 = 0; q0 < 16 * CPR; q0 += 64) {
          const int q = q0 + lane, rl = q / CPR, ch = q - rl * CPR, row = 16 * r + rl;
          if (q < 16 * CPR && row < cnt && ((okmask >> ((ch * (16 / ES)) >> 4)) & 1u)) {
            const uint4 v = *reinterpret_cast<const uint4*>(mine + rl * OROW + ch * 16);
            *reinterpret_cast<uint4*>(obytes + ((size_t)dst_rows[row] * N + col0 + ch * (16 / ES)) * ES) = v;
          }
        }
      }
      return;
    }
    // a lane holds row 16 r + c, columns 4 kq + (0..3) of each of the wave's 16-column tiles (ocol: the lane's column c
    // of the tile, so the tile begins at ocol - c; for the dense weight jok says the lane's column exists, and with N a
    // multiple of 4 the tile's columns from 4 kq on exist or not together)
    const bool whole = N % 4 == 0;
#pragma unroll
    for (int r = 0; r < RT; ++r) {
      const int row = 16 * r + c;
      if (row >= cnt) continue;
      const size_t base = (size_t)dst_rows[row] * N;
#pragma unroll
      for (int j = 0; j < (NM == 2 ? TJ / 2 : TJ); ++j) {
        const int col = ocol[j] - c + 4 * kq;
        if (!tile_ok[j]) continue;
        float a4[4], u4[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          a4[i] = acc[j][r][i] * UNSCALE;
          u4[i] = NM == 2 ? acc[j + TJ / 2][r][i] * UNSCALE : 0.f;
        }
        store4<EPI>(out, base + col, a4, u4, limit, N - col, whole);
      }
    }
    return;
  }
  // D[row 4 kq + i][column c] of each 16 x 16 tile
#pragma unroll
  for (int r = 0; r < RT; ++r) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int row = 16 * r + 4 * kq + i;
      if (row >= cnt) continue;
      const size_t base = (size_t)dst_rows[row] * N;
      if constexpr (NM == 2) {
#pragma unroll
        for (int j = 0; j < TJ / 2; ++j)
          if (jok[j])
            store_out<EPI>(out, base + ocol[j], acc[j][r][i] * UNSCALE, acc[j + TJ / 2][r][i] * UNSCALE, limit);
      } else {
#pragma unroll
        for (int j = 0; j < TJ; ++j)
          if (jok[j]) store_out<EPI>(out, base + ocol[j], acc[j][r][i] * UNSCALE, 0.f, limit);
      }
    }
  }
}

// 32-column blocks a workgroup of the big kernel covers
constexpr int big_blocks(int nm) { return nm == 2 ? BIG_WAVES : 2 * BIG_WAVES; }

template <int GS, int NM, int EPI, int AR>
__global__ void __launch_bounds__(BIG_THREADS, 1)
    experts_prefill_big_kernel(const uint16_t* __restrict__ X, int64_t x_stride, int slots,
                               const uint32_t* __restrict__ W, int KG, int NB, const int* __restrict__ items,
                               const int* __restrict__ counts, const int* __restrict__ members,
                               void* __restrict__ out, int N, float limit) {
  constexpr int BW = block_words(GS);
  constexpr int NBW = big_blocks(NM);
  extern __shared__ __align__(16) unsigned char smem[];
  __shared__ int src_rows[BIG_ROWS], dst_rows[BIG_ROWS];
  const int nbt = (NB + NBW - 1) / NBW;
  const int it = blockIdx.x / nbt, cbt = blockIdx.x - it * nbt;
  TF_MARK(0);
  if (it >= counts[0]) return;
  const int e = items[3 * it], first = items[3 * it + 1], cnt = min(items[3 * it + 2], BIG_ROWS);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, c = lane & 15, kq = lane >> 4;
  if (tid < BIG_ROWS) {
    const int p = members[first + (tid < cnt ? tid : 0)];
    dst_rows[tid] = p;
    src_rows[tid] = slots ? p / slots : p;
  }
  __syncthreads();
  TF_MARK(1);
  // the wave's four B operands: (matrix, 32-column block, 16-column half)
  const uint32_t* We = W + (size_t)e * NB * KG * (size_t)(NM * BW);      // the expert's matrices (wave-uniform)
  ExpertSource<GS, NM> ws;
  ws.rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint32_t*>(We), 0, (uint32_t)NB * KG * (NM * BW) * 4u, 0x00020000);
  int ocol[4];
  bool jok[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int nb = NM == 2 ? cbt * NBW + wave : cbt * NBW + wave * 2 + (j >> 1);
    jok[j] = nb < NB;
    ocol[j] = nb * 32 + (j & 1) * 16 + c;
  }
  {
    // the column this lane loads: column lane & 31 of block (matrix or neighbour) lane >> 5
    const int m = NM == 2 ? lane >> 5 : 0;
    const int nb = min(NM == 2 ? cbt * NBW + wave : cbt * NBW + wave * 2 + (lane >> 5), NB - 1);
    const uint32_t blk = (uint32_t)(nb * KG) * (uint32_t)(NM * BW) + m * BW;
    ws.qp = (blk + (lane & 31) * 4) * 4u;
    ws.sp = (blk + 32 * GS / 8 + (lane & 31)) * 4u;
  }
  // one matrix (the down projection, whose outputs are the bulk of a chunk's stores): tiles weights-first and whole
  // lines out through LDS (4 % of the launch); gate and up with the SwiGLU between them: neither (3 % the other way)
  constexpr bool OUT_LINES = NM == 1;
  const int K = KG * GS;
  if (cnt <= 32) big_body<GS, NM, EPI, 2, AR, OUT_LINES, ExpertSource<GS, NM>, 4, BIG_THREADS, OUT_LINES>(X, x_stride, ws, ocol, jok, K, src_rows, dst_rows, cnt, out, N, limit, smem);
  else if (cnt <= 64) big_body<GS, NM, EPI, 4, AR, OUT_LINES, ExpertSource<GS, NM>, 4, BIG_THREADS, OUT_LINES>(X, x_stride, ws, ocol, jok, K, src_rows, dst_rows, cnt, out, N, limit, smem);
  else big_body<GS, NM, EPI, 8, AR, OUT_LINES, ExpertSource<GS, NM>, 4, BIG_THREADS, OUT_LINES>(X, x_stride, ws, ocol, jok, K, src_rows, dst_rows, cnt, out, N, limit, smem);
  TF_MARK(4);
#ifdef TF_TIMELINE
  __builtin_amdgcn_s_waitcnt(0);         // mark 5 is the results written, not only issued
#endif
  TF_MARK(5);
}

// The same units taken by workgroups that stay, one a compute unit (a unit = an item's 512 weight columns, as a
// workgroup of experts_prefill_big_kernel takes).  A workgroup has a compute unit to itself (the body's registers), so
// in the kernel above nothing runs under a unit's head (the item's rows looked up through two dependent reads, then
// the first operands' trip), its results' drain, and the dispatch of the next workgroup; and with five or six
// workgroups of 47 to 67 us to a compute unit, those that got five sit idle for the last tenth of the launch.  Here
//   * the units are walked in one order, place q = 0, 1, 2, ...: workgroup w of G takes places w and w + G, then
//     whichever place is next on a ticket counter in memory (an atomic add that returns: ticket t is place 2 G + t),
//     so a compute unit that finishes early takes more and the launch ends within a unit's time of the moment the
//     work runs out;
//   * the walk takes two units from the plan's front (the full items, bound by the matrix cores) for each one from
//     its back (the short items, which mostly stream their expert's tables), so both kinds run side by side and
//     the long units are dealt out in the launch's first three fifths: what is left for its end is short;
//   * everything a unit needs to begin is fetched under the units before it: at a unit's top the workgroup requests
//     the next unit's row list and the ticket for the unit after that; both have arrived (for nothing: a wave's
//     memory operations complete in issue order) when the first operands have, where the rows go to LDS and wave 0
//     requests the ticket's item, which it holds through the loop over K and puts into LDS at the unit's end.
// The ticket counter is zero between launches: F = max(total - 2 G, 0) + clamp(total - G, 0, G) tickets are drawn in a
// launch over `total` units (every workgroup whose second unit exists draws until its first ticket past the end),
// and the thread that draws ticket F - 1 puts the counter back.  Launches that share a counter must not overlap.
// Same units, same body, same bits.
//
// The rows' lists and the next item live behind the activation and weight stages in the dynamic LDS:
// [unit parity][source row, pair][row of the item], then (expert, first member, rows, unit).
constexpr int RESIDENT_LDS = BIG_LDS + 2 * 2 * BIG_ROWS * 4 + 16;

__device__ __forceinline__ int* resident_rows(int parity, int which) {
  extern __shared__ __align__(16) unsigned char smem[];
  return reinterpret_cast<int*>(smem + BIG_LDS) + (parity * 2 + which) * BIG_ROWS;
}

template <int GS, int NM, int EPI, int AR, int RT, class STAGED>
__device__ __forceinline__ void resident_unit(const uint16_t* __restrict__ X, int64_t x_stride,
                                              const uint32_t* __restrict__ We, int KG, int NB, int cbt, int cnt,
                                              void* __restrict__ out, int N, float limit, int parity, int tid,
                                              STAGED& staged) {
  constexpr int BW = block_words(GS);
  constexpr int NBW = big_blocks(NM);
  extern __shared__ __align__(16) unsigned char smem[];
  const int lane = tid & 63, wave = tid >> 6, c = lane & 15, kq = lane >> 4;
  ExpertSource<GS, NM> ws;
  ws.rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint32_t*>(We), 0, (uint32_t)NB * KG * (NM * BW) * 4u, 0x00020000);
  int ocol[4];
  bool jok[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int nb = NM == 2 ? cbt * NBW + wave : cbt * NBW + wave * 2 + (j >> 1);
    jok[j] = nb < NB;
    ocol[j] = nb * 32 + (j & 1) * 16 + c;
  }
  {
    // the column this lane loads: column lane & 31 of block (matrix or neighbour) lane >> 5
    const int m = NM == 2 ? lane >> 5 : 0;
    const int nb = min(NM == 2 ? cbt * NBW + wave : cbt * NBW + wave * 2 + (lane >> 5), NB - 1);
    const uint32_t blk = (uint32_t)(nb * KG) * (uint32_t)(NM * BW) + m * BW;
    ws.qp = (blk + (lane & 31) * 4) * 4u;
    ws.sp = (blk + 32 * GS / 8 + (lane & 31)) * 4u;
  }
  constexpr bool OUT_LINES = NM == 1;
  big_body<GS, NM, EPI, RT, AR, OUT_LINES, ExpertSource<GS, NM>, 4, BIG_THREADS, OUT_LINES>(
      X, x_stride, ws, ocol, jok, KG * GS, resident_rows(parity, 0), resident_rows(parity, 1), cnt, out, N, limit, smem,
      staged, tid);
}

template <int GS, int NM, int EPI, int AR>
__global__ void __launch_bounds__(BIG_THREADS, 1)
    experts_prefill_resident_kernel(const uint16_t* __restrict__ X, int64_t x_stride, int slots,
                                    const uint32_t* __restrict__ W, int KG, int NB, const int* __restrict__ items,
                                    const int* __restrict__ counts, int* __restrict__ ticket,
                                    const int* __restrict__ members, void* __restrict__ out, int N, float limit) {
  constexpr int BW = block_words(GS);
  constexpr int NBW = big_blocks(NM);
  const int nbt = (NB + NBW - 1) / NBW;
  const int total = counts[0] * nbt, G = gridDim.x;
  // place q of the walk -> unit: two from the front of the plan (full items: matrix work), then one from its back
  // (the experts' short last items: mostly their tables' trip from memory), so that the two kinds run side by side
  // instead of one after the other (one for one: the up launch 316-322 us where this order takes 306-319)
  auto unit_at = [&](int q) { const int t = q / 3, r = q - 3 * t; return r == 2 ? total - 1 - t : 2 * t + r; };
  const int tickets = max(total - 2 * G, 0) + min(max(total - G, 0), G);
  int tid = threadIdx.x;
  int unit = blockIdx.x;
  if (unit >= total) return;
  int* next_item = resident_rows(2, 0);
  // an item's (expert, first member, rows): the same for every thread
  auto item_of = [&](int u, int& e, int& first, int& cnt) {
    const int it = unit_at(min(u, total - 1)) / nbt;
    e = __builtin_amdgcn_readfirstlane(items[3 * it]);
    first = __builtin_amdgcn_readfirstlane(items[3 * it + 1]);
    cnt = min(__builtin_amdgcn_readfirstlane(items[3 * it + 2]), BIG_ROWS);
  };
  int unit1 = unit + G, e, first, cnt, e1, first1, cnt1;
  item_of(unit, e, first, cnt);
  item_of(unit1, e1, first1, cnt1);
  if (tid < BIG_ROWS) {
    const int p = members[first + (tid < cnt ? tid : 0)];
    resident_rows(0, 1)[tid] = p;
    resident_rows(0, 0)[tid] = slots ? p / slots : p;
  }
  __syncthreads();
  for (int k = 0;; ++k) {
    // what a unit derives from the thread's number is derived again for every unit: kept across units instead, it
    // would crowd the body's registers
    asm volatile("" : "+v"(tid));
    TF_MARK(0);
    TF_MARK(1);
    const int it = unit_at(unit) / nbt, cbt = unit_at(unit) - it * nbt;
    const int more = unit1 < total;
    // requested now, used once this unit's first operands are here: the next unit's rows, the ticket after it
    int p1 = 0, held = 0;
    if (more && tid < BIG_ROWS) p1 = members[first1 + (tid < cnt1 ? tid : 0)];
    if (more && tid == 0) held = __hip_atomic_fetch_add(ticket, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    auto staged = [&]() {
      if (!more) return;
      if (tid < BIG_ROWS) {
        resident_rows(1 - (k & 1), 1)[tid] = p1;
        resident_rows(1 - (k & 1), 0)[tid] = slots ? p1 / slots : p1;
      }
      if (tid < 64) {
        // wave 0: the ticket's unit and its item, three ints on their way through the loop over K
        if (tid == 0 && held == tickets - 1) __hip_atomic_store(ticket, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const int u2 = 2 * G + __builtin_amdgcn_readfirstlane(held);
        held = tid < 3 ? items[3 * (unit_at(min(u2, total - 1)) / nbt) + tid] : u2;
      }
    };
    const uint32_t* We = W + (size_t)e * NB * KG * (size_t)(NM * BW);
    if (cnt <= 32) resident_unit<GS, NM, EPI, AR, 2>(X, x_stride, We, KG, NB, cbt, cnt, out, N, limit, k & 1, tid, staged);
    else if (cnt <= 64) resident_unit<GS, NM, EPI, AR, 4>(X, x_stride, We, KG, NB, cbt, cnt, out, N, limit, k & 1, tid, staged);
    else resident_unit<GS, NM, EPI, AR, 8>(X, x_stride, We, KG, NB, cbt, cnt, out, N, limit, k & 1, tid, staged);
    TF_MARK(4);
#ifdef TF_TIMELINE
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#endif
    TF_MARK_AS(5, unit_at(unit));
    if (!more) break;
    if (tid < 4) next_item[tid] = held;
    __syncthreads();          // every wave is done with the stages (and its results' corner of them) and this unit's rows
    unit = unit1, e = e1, first = first1, cnt = cnt1;
    e1 = __builtin_amdgcn_readfirstlane(next_item[0]);
    first1 = __builtin_amdgcn_readfirstlane(next_item[1]);
    cnt1 = min(__builtin_amdgcn_readfirstlane(next_item[2]), BIG_ROWS);
    unit1 = __builtin_amdgcn_readfirstlane(next_item[3]);
  }
}

// The dense prompt matmul on the same pipeline: 128 rows x 512 columns a workgroup, a wave a 64-column tile.
template <int GS, int EPI, int AR>
__global__ void __launch_bounds__(BIG_THREADS, 1)
    qmm_prefill_big_kernel(const uint16_t* __restrict__ X, int64_t ldx, const uint32_t* __restrict__ W,
                           const uint16_t* __restrict__ S, const uint16_t* __restrict__ B, void* __restrict__ out,
                           int M, int N, int KG, int npad) {
  extern __shared__ __align__(16) unsigned char smem[];
  __shared__ int rows[BIG_ROWS];
  const int ct = (N + 511) >> 9;
  const int rt = blockIdx.x / ct, cbt = blockIdx.x - rt * ct;
  const int m0 = rt * BIG_ROWS, cnt = min(BIG_ROWS, M - m0);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, c = lane & 15, kq = lane >> 4;
  TF_MARK(0);
  if (tid < BIG_ROWS) rows[tid] = m0 + (tid < cnt ? tid : 0);
  __syncthreads();
  TF_MARK(1);
  const int tiles = npad >> 6, tile = cbt * 8 + wave;
  const bool ok = tile < tiles;
  DenseSource<GS> ws;
  ws.codes = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint32_t*>(W), 0, (uint32_t)tiles * KG * (GS / 32) * 1024u, 0x00020000);
  ws.scales = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(S), 0, (uint32_t)KG * npad * 2u, 0x00020000);
  ws.biases = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(B), 0, (uint32_t)KG * npad * 2u, 0x00020000);
  ws.row_bytes = npad * 2;
  int ocol[4];
  bool jok[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int col = (ok ? tile : 0) * 64 + 16 * j + c;      // columns up to npad are stored zeros
    ocol[j] = col;
    jok[j] = ok && col < N;
  }
  ws.qp = ((uint32_t)(ok ? tile : 0) * KG * (GS / 32) * 256u + lane * 4) * 4u;      // the column this lane loads: lane
  ws.cp = ((ok ? tile : 0) * 64 + lane) * 2;
  const int K = KG * GS;
  if (cnt <= 32) big_body<GS, 1, EPI, 2, AR, true>(X, ldx, ws, ocol, jok, K, rows, rows, cnt, out, N, 0.f, smem);
  else if (cnt <= 64) big_body<GS, 1, EPI, 4, AR, true>(X, ldx, ws, ocol, jok, K, rows, rows, cnt, out, N, 0.f, smem);
  else big_body<GS, 1, EPI, 8, AR, true>(X, ldx, ws, ocol, jok, K, rows, rows, cnt, out, N, 0.f, smem);
  TF_MARK(4);
#ifdef TF_TIMELINE
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#endif
  TF_MARK(5);
}

// ---- dense prompt matmul --------------------------------------------------------------------------------------------

template <int GS>
struct LaneWords {
  const uint32_t* base;      // the lane's 64-column tile: + (32 * half + c) * 4 + kq applied
  const uint16_t* S;
  const uint16_t* B;
  int64_t stride;
  int KG;
  __device__ __forceinline__ uint32_t word(int g, int, int i, int t) const {
    return base[((size_t)g * (GS / 32) + i) * 256 + t * 64];
  }
  __device__ __forceinline__ uint32_t sb(int g, int, int t) const {
    return (uint32_t)S[(size_t)g * stride + t * 16] | ((uint32_t)B[(size_t)g * stride + t * 16] << 16);
  }
};

template <int GS, int EPI, int RT, int AR>
__global__ void __launch_bounds__(256)
    qmm_prefill_kernel(const uint16_t* __restrict__ X, int64_t ldx, const uint32_t* __restrict__ W,
                       const uint16_t* __restrict__ S, const uint16_t* __restrict__ B, void* __restrict__ out, int M,
                       int N, int KG, int npad) {
  extern __shared__ __align__(16) unsigned char smem[];
  __shared__ int rows[16 * RT];
  const int ct = (N + 127) >> 7;
  const int rt = blockIdx.x / ct, cbt = blockIdx.x - rt * ct;
  const int m0 = rt * 16 * RT, cnt = min(16 * RT, M - m0);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, c = lane & 15, kq = lane >> 4;
  if (tid < 16 * RT) rows[tid] = m0 + (tid < cnt ? tid : 0);
  __syncthreads();
  const int col0 = cbt * 128 + wave * 32;
  const bool ok = col0 < N;                      // columns up to npad are stored zeros, safe to read
  const int tile = (ok ? col0 : 0) >> 6, half = (col0 >> 5) & 1;
  LaneWords<GS> ws;
  ws.base = W + ((size_t)tile * KG) * (size_t)(GS / 32 * 256) + (32 * half + c) * 4 + kq;
  ws.S = S + (ok ? col0 : 0) + c;
  ws.B = B + (ok ? col0 : 0) + c;
  ws.stride = npad;
  ws.KG = KG;
  mfma_body<GS, 1, EPI, RT, AR, true>(X, ldx, KG * GS, ws, rows, cnt, out, N, col0, ok, rows, 0.f, smem);
}

template <int RT>
constexpr size_t stage_bytes() {
  return 2 * (size_t)(16 * RT) * AROW;
}

// compute units of the current device (looked up once a device)
int compute_units() {
  static int cached[64] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  if (!cached[dev]) {
    hipDeviceProp_t prop;
    cached[dev] = hipGetDeviceProperties(&prop, dev) == hipSuccess && prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
  }
  return cached[dev];
}

template <int GS, int NM, int EPI>
int launch_experts_prefill(int tile, int arith, const uint16_t* x, int64_t x_stride, int slots, const uint32_t* w,
                           int kg, int nb, const int* items, int* counts, const int* members, void* out, int n,
                           float limit, int64_t max_items, hipStream_t s) {
  const int64_t grid = max_items * ((nb + 3) / 4);
  if (grid < 1) return 0;
  TF_REQUIRE(grid <= 0x7FFFFFFF, "experts: %lld workgroups exceed the grid limit", (long long)grid);
  const dim3 g((unsigned)grid), b(256);
#define TF_SMALL(RT_, AR_)                                                                                              \
  experts_prefill_kernel<GS, NM, EPI, RT_, AR_><<<g, b, stage_bytes<RT_>(), s>>>(x, x_stride, slots, w, kg, nb, items, \
                                                                               counts, members, out, n, limit)
  if (tile == 16) {
    if (arith) TF_SMALL(1, 1);
    else TF_SMALL(1, 0);
  } else if ((kg * GS) % KSTEP) {
    // a K that is not whole steps of 64 (odd group counts at g32): the small kernel's tail handling
    if (tile == 64) {
      if (arith) TF_SMALL(4, 1);
      else TF_SMALL(4, 0);
    } else {
      if (arith) TF_SMALL(8, 1);
      else TF_SMALL(8, 0);
    }
  } else {
    constexpr int NBW = big_blocks(NM);
    const int64_t big = max_items * ((nb + NBW - 1) / NBW);
    TF_REQUIRE(big <= 0x7FFFFFFF, "experts: %lld workgroups exceed the grid limit", (long long)big);
    // workgroups that stay and walk the units by stride, one a compute unit, once there are units to walk
    const int cus = compute_units();
    if (big > 2 * cus) {
      const dim3 rg((unsigned)cus);
      if (arith)
        experts_prefill_resident_kernel<GS, NM, EPI, 1><<<rg, BIG_THREADS, RESIDENT_LDS, s>>>(
            x, x_stride, slots, w, kg, nb, items, counts, counts + 2, members, out, n, limit);
      else
        experts_prefill_resident_kernel<GS, NM, EPI, 0><<<rg, BIG_THREADS, RESIDENT_LDS, s>>>(
            x, x_stride, slots, w, kg, nb, items, counts, counts + 2, members, out, n, limit);
      TF_LAUNCH_OK("tf_experts_prefill");
      return 0;
    }
    const dim3 bg((unsigned)big);
    if (arith)
      experts_prefill_big_kernel<GS, NM, EPI, 1><<<bg, BIG_THREADS, BIG_LDS, s>>>(
          x, x_stride, slots, w, kg, nb, items, counts, members, out, n, limit);
    else
      experts_prefill_big_kernel<GS, NM, EPI, 0><<<bg, BIG_THREADS, BIG_LDS, s>>>(
          x, x_stride, slots, w, kg, nb, items, counts, members, out, n, limit);
  }
#undef TF_SMALL
  TF_LAUNCH_OK("tf_experts_prefill");
  return 0;
}

// tile: 0 = chosen from the row count; 1, 4, 8 = the four-wave kernel on 16, 64 or 128 rows a workgroup; 9 = the
// eight-wave kernel (128 rows x 512 columns; K in whole steps of 64).  The same bits whatever the tile.
template <int GS, int EPI>
int launch_qmm_prefill(int arith, int tile, const uint16_t* x, int64_t ldx, const uint32_t* w, const uint16_t* s,
                       const uint16_t* b, void* out, int m, int n, int kg, hipStream_t st) {
  const int npad = (n + 127) / 128 * 128;
  const int ct = (n + 127) / 128;
#define TF_SMALL(RT_, AR_)                                                                                       \
  qmm_prefill_kernel<GS, EPI, RT_, AR_><<<(unsigned)(((m + 16 * RT_ - 1) / (16 * RT_)) * ct), 256, stage_bytes<RT_>(), \
                                          st>>>(x, ldx, w, s, b, out, m, n, kg, npad)
  TF_REQUIRE((int64_t)((m + 15) / 16) * ct <= 0x7FFFFFFF, "qmm_prefill: grid too large");
  const bool big_ok = (kg * GS) % KSTEP == 0 && (int64_t)npad * kg * GS / 2 < (1ll << 32);
  TF_REQUIRE(tile != 9 || big_ok, "qmm_prefill: tile 9 (the eight-wave kernel) takes K in whole steps of 64");
  const int rows = tile == 1 ? 16 : tile == 4 ? 64 : tile == 8 ? 128 : tile == 9 ? 129 : m;     // as if this many rows
  if (rows <= 16) {
    if (arith) TF_SMALL(1, 1);
    else TF_SMALL(1, 0);
  } else if (rows <= 64) {
    if (arith) TF_SMALL(4, 1);
    else TF_SMALL(4, 0);
  } else if (big_ok && tile != 8) {
    const unsigned grid = (unsigned)((int64_t)((m + BIG_ROWS - 1) / BIG_ROWS) * ((n + 511) / 512));
    if (arith)
      qmm_prefill_big_kernel<GS, EPI, 1><<<grid, BIG_THREADS, BIG_LDS, st>>>(x, ldx, w, s, b, out, m, n, kg, npad);
    else
      qmm_prefill_big_kernel<GS, EPI, 0><<<grid, BIG_THREADS, BIG_LDS, st>>>(x, ldx, w, s, b, out, m, n, kg, npad);
  } else if (arith) {
    TF_SMALL(8, 1);
  } else {
    TF_SMALL(8, 0);
  }
#undef TF_SMALL
  TF_LAUNCH_OK("tf_qmm_prefill");
  return 0;
}

}  // namespace
}  // namespace tf

using namespace tf;

TF_TIMELINE_EXPORT(prefill)

extern "C" int tf_experts_prefill(int gs, int epi, const uint16_t* x, int64_t x_stride, int slots, const uint32_t* w,
                                  int kg, int nb, const int32_t* items, int32_t* counts, const int32_t* members,
                                  void* out, int n, float limit, int64_t max_items, int tile, int arith,
                                  tf_stream_t stream) {
  clear_error();
  TF_REQUIRE(arith == TF_ARITH_F16 || arith == TF_ARITH_BF16, "prefill arithmetic %d: TF_ARITH_F16 or TF_ARITH_BF16", arith);
  TF_REQUIRE(gs == 32 || gs == 64, "experts: groups of 32 or 64 inputs, not %d", gs);
  TF_REQUIRE(x && w && items && counts && members && out, "experts: null pointer argument");
  TF_REQUIRE(kg >= 1 && nb >= 1 && n == nb * 32, "experts: n (%d) must be the column blocks (%d) times 32", n, nb);
  TF_REQUIRE(aligned16(x) && x_stride % 8 == 0, "x: rows of K = groups * group size inputs, 16-byte aligned");
  TF_REQUIRE(tile == 16 || tile == 64 || tile == 128, "prefill items hold 16, 64 or 128 pairs, not %d", tile);
  TF_REQUIRE(slots >= 0 && max_items >= 0, "experts: negative slots or max_items");
  hipStream_t s = as_stream(stream);
#define TF_PRE(GS_, NM_, EPI_) \
  if (gs == GS_ && epi == EPI_) \
    return launch_experts_prefill<GS_, NM_, EPI_>(tile, arith, x, x_stride, slots, w, kg, nb, items, counts, members, out, n, limit, max_items, s);
  TF_PRE(32, 1, 0) TF_PRE(32, 1, 1) TF_PRE(32, 1, 3) TF_PRE(32, 1, 4) TF_PRE(32, 2, 2)
  TF_PRE(64, 1, 0) TF_PRE(64, 1, 1) TF_PRE(64, 1, 3) TF_PRE(64, 1, 4) TF_PRE(64, 2, 2)
#undef TF_PRE
  set_error("experts: no prefill kernel for group %d and epilogue %d", gs, epi);
  return 1;
}

extern "C" int tf_qmm_prefill(const uint16_t* x, int64_t ldx, const uint32_t* weight, const uint16_t* scales,
                              const uint16_t* biases, void* out, int m, int n, int k, int gs, int f32, int tile,
                              int arith, tf_stream_t stream) {
  clear_error();
  TF_REQUIRE(arith == TF_ARITH_F16 || arith == TF_ARITH_BF16, "prefill arithmetic %d: TF_ARITH_F16 or TF_ARITH_BF16", arith);
  TF_REQUIRE(gs == 32 || gs == 64, "groups of 32 or 64");
  TF_REQUIRE(tile == 0 || tile == 1 || tile == 4 || tile == 8 || tile == 9, "qmm_prefill: tile 0 (chosen from the row count), 1, 4, 8 or 9, not %d", tile);
  TF_REQUIRE(x && weight && scales && biases && out && m >= 1 && n >= 1, "qmm_prefill: null pointer or empty shape");
  TF_REQUIRE(aligned16(x) && (m == 1 || ldx % 8 == 0), "x rows must start on 16-byte boundaries");
  TF_REQUIRE(k >= gs && k % gs == 0, "K splits into whole groups");
  hipStream_t s = as_stream(stream);
  const int kg = k / gs;
  if (gs == 64) return f32 ? launch_qmm_prefill<64, 0>(arith, tile, x, ldx, weight, scales, biases, out, m, n, kg, s)
                           : launch_qmm_prefill<64, 3>(arith, tile, x, ldx, weight, scales, biases, out, m, n, kg, s);
  return f32 ? launch_qmm_prefill<32, 0>(arith, tile, x, ldx, weight, scales, biases, out, m, n, kg, s)
             : launch_qmm_prefill<32, 3>(arith, tile, x, ldx, weight, scales, biases, out, m, n, kg, s);
}
