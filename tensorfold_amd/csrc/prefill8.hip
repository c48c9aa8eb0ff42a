// The FP8 prompt path of the dense 4-bit matmul (tf_quantize_rows, tf_qmm_prefill8): what the reference's
// kernels/qmm.py:222-268 (`quantize_rows`, `prefill_matmul8`) and kernels/qmm_prefill8.cu do.
//
//   quantize_rows   a row's scale a = max|x| / 448 (1 for a row of zeros), x8 = e4m3(x / a), xs[g] = bf16(sum of the
//                   group's inputs / a)
//   prefill8        per group, in order:  acc = fma(P, s, acc),  P = sum over the group of x8 * q  (exact operands:
//                   a 4-bit code is an e4m3 number), then acc += xs . bias over the groups (bf16 MFMAs), then * a
//
// A nibble in a byte IS the e4m3 number q * 2^-9 (a subnormal below 8, exponent field 1 from 8 on), so the B operand of
// v_mfma_f32_16x16x32_fp8_fp8 is the packed word's low nibbles and its high nibbles, two vector instructions a word;
// the 2^9 rides in the scale (a power of two: the fma's rounding does not move).  The eight inputs a lane holds come
// out in the order (0, 4, 1, 5, 2, 6, 3, 7) of their octet; quantize_rows writes x8 in that order, so the A operand is
// eight bytes as they lie in the row.  A row's bits depend on that row alone: whole steps of 64 inputs, no K split,
// a 16-row MFMA tile keeps rows apart.
//
// A workgroup of eight waves takes 128 rows x 256 columns; a wave 32 columns (two B operands) and every row tile: 64
// accumulator registers (four B operands a wave, 128 accumulator registers, did not fit beside the group's partial
// sums: the compiler spilled the weights' registers inside the loop).  x8 is staged through LDS (80-byte rows, two stages, one barrier a step of 64 inputs), the packed words come straight
// into registers two steps ahead, as in the 16-bit prompt kernel (prefill.hip).

#include "tf_common.h"

namespace tf {
namespace {

constexpr int P8_ROWS = 128, P8_WAVES = 8, P8_THREADS = P8_WAVES * 64, P8_KSTEP = 64;
constexpr int P8_TJ = 2;                        // 16-column tiles a wave
constexpr int P8_AROW = P8_KSTEP + 16;          // bytes of an LDS row: 64 e4m3 inputs, 16 of padding
constexpr int P8_STAGE = P8_ROWS * P8_AROW;

typedef __attribute__((ext_vector_type(2))) uint32_t u32x2_t;

__device__ __forceinline__ long as_long(uint32_t lo, uint32_t hi) {
  const u32x2_t v = {lo, hi};
  return __builtin_bit_cast(long, v);
}

// ---- quantize_rows ---------------------------------------------------------------------------------------------------
//
// A workgroup a row.  The row's largest magnitude first, then a thread an octet of inputs: eight divisions, eight
// conversions (round to nearest even, the hardware's), the bytes stored in operand order, and the octet's sum in input
// order; the first lane of a group then adds the group's octet sums in order.  Sums are of the inputs themselves, not
// of the quantized values (kernels/qmm.py:241-243).
template <int GS>
__global__ void __launch_bounds__(256)
    quantize_rows_kernel(const uint16_t* __restrict__ X, int64_t ldx, int K, uint8_t* __restrict__ X8,
                         uint16_t* __restrict__ XS, float* __restrict__ A) {
  __shared__ float wmax[4];
  const int row = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const uint16_t* x = X + (size_t)row * ldx;
  const int octets = K / 8;
  float top = 0.f;
  for (int o = tid; o < octets; o += 256) {
    const uint4 v = *reinterpret_cast<const uint4*>(x + 8 * o);
    const uint32_t d[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) top = fmaxf(top, fmaxf(fabsf(bf16_lo(d[i])), fabsf(bf16_hi(d[i]))));
  }
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) top = fmaxf(top, __shfl_xor(top, m));
  if (lane == 0) wmax[wave] = top;
  __syncthreads();
  top = fmaxf(fmaxf(wmax[0], wmax[1]), fmaxf(wmax[2], wmax[3]));
  const float a = top > 0.f ? __fdiv_rn(top, 448.f) : 1.f;
  if (tid == 0) A[row] = a;
  constexpr int OPG = GS / 8;                     // octets a group: 4 or 8 neighbouring lanes
  for (int o0 = 0; o0 < octets; o0 += 256) {
    const int o = o0 + tid;
    float s = 0.f;
    if (o < octets) {
      const uint4 v = *reinterpret_cast<const uint4*>(x + 8 * o);
      const uint32_t d[4] = {v.x, v.y, v.z, v.w};
      float f[8];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        f[2 * i] = bf16_lo(d[i]);
        f[2 * i + 1] = bf16_hi(d[i]);
      }
#pragma unroll
      for (int i = 0; i < 8; ++i) s += f[i];
      float q[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) q[i] = __fdiv_rn(f[i], a);
      // bytes in operand order: inputs (0, 4, 1, 5) then (2, 6, 3, 7)
      int lo = 0, hi = 0;
      lo = __builtin_amdgcn_cvt_pk_fp8_f32(q[0], q[4], lo, false);
      lo = __builtin_amdgcn_cvt_pk_fp8_f32(q[1], q[5], lo, true);
      hi = __builtin_amdgcn_cvt_pk_fp8_f32(q[2], q[6], hi, false);
      hi = __builtin_amdgcn_cvt_pk_fp8_f32(q[3], q[7], hi, true);
      *reinterpret_cast<uint2*>(X8 + (size_t)row * K + 8 * o) = make_uint2((uint32_t)lo, (uint32_t)hi);
    }
    // the group's octet sums, in order, into its first lane (a group's lanes are neighbours inside a wave)
    float g = s;
#pragma unroll
    for (int j = 1; j < OPG; ++j) g += __shfl_down(s, j);
    if (o < octets && (tid % OPG) == 0) XS[(size_t)row * (K / GS) + o / OPG] = (uint16_t)f32_bf16_bits(__fdiv_rn(g, a));
  }
}

// ---- prefill8 --------------------------------------------------------------------------------------------------------

template <int GS, bool F32, int RT>
__device__ __forceinline__ void prefill8_body(const uint8_t* __restrict__ X8, const uint16_t* __restrict__ XS,
                                              const float* __restrict__ A, const __amdgpu_buffer_rsrc_t codes,
                                              const __amdgpu_buffer_rsrc_t scales, const uint16_t* __restrict__ B,
                                              void* __restrict__ out, int m0, int cnt, int N, int K, int KG, int npad,
                                              const uint32_t (&wp)[P8_TJ], const uint32_t (&cp)[P8_TJ], const int (&ocol)[P8_TJ],
                                              const bool (&jok)[P8_TJ], unsigned char* smem) {
  constexpr int CPG = GS / 32;                  // 32-input chunks a group
  constexpr int GPS = P8_KSTEP / GS;            // groups a step
  const int tid = threadIdx.x, lane = tid & 63, c = lane & 15, kq = lane >> 4;
  const int steps = K / P8_KSTEP, last = steps - 1;
  // this thread's 16-byte piece of a step's x8 tile: (row tid / 4, piece tid % 4); rows past the tile repeat its last
  const int prow = tid >> 2, piece = tid & 3;
  const uint8_t* asrc = X8 + (size_t)(m0 + min(prow, cnt - 1)) * K + piece * 16;
  const bool astage = prow < 16 * RT;
  unsigned char* adst = smem + prow * P8_AROW + piece * 16;
  auto load_a = [&](int step) { return astage ? *reinterpret_cast<const uint4*>(asrc + (size_t)step * P8_KSTEP) : make_uint4(0, 0, 0, 0); };
  auto store_a = [&](int buf, const uint4& v) {
    if (astage) *reinterpret_cast<uint4*>(adst + buf * P8_STAGE) = v;
  };
  // the lane's packed word of each column tile and chunk of a step, and its columns' stored scales (bf16 bits)
  auto load_w = [&](int step, uint32_t (&w)[P8_TJ][2], uint32_t (&s)[P8_TJ][GPS]) {
    const int soff = step * 2048;               // a step is two chunks of 1 KB a 64-column tile
#pragma unroll
    for (int j = 0; j < P8_TJ; ++j) {
#pragma unroll
      for (int i = 0; i < 2; ++i) w[j][i] = __builtin_amdgcn_raw_buffer_load_b32(codes, wp[j] + i * 1024, soff, 0);
#pragma unroll
      for (int gi = 0; gi < GPS; ++gi)
        s[j][gi] = __builtin_amdgcn_raw_buffer_load_b16(scales, cp[j], (step * GPS + gi) * npad * 2, 0);
    }
  };

  f32x4_t acc[P8_TJ][RT];
#pragma unroll
  for (int j = 0; j < P8_TJ; ++j)
#pragma unroll
    for (int r = 0; r < RT; ++r) acc[j][r] = (f32x4_t){0.f, 0.f, 0.f, 0.f};

  uint32_t wr[2][P8_TJ][2], sr[2][P8_TJ][GPS];
  load_w(0, wr[0], sr[0]);
  uint4 ar = load_a(0);
  load_w(min(1, last), wr[1], sr[1]);
  store_a(0, ar);
  __syncthreads();
  for (int step0 = 0; step0 < steps; step0 += 2) {
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int step = step0 + u;
      if (step < steps) {
        ar = load_a(min(step + 1, last));
        const unsigned char* abuf = smem + u * P8_STAGE + c * P8_AROW + kq * 8;
#pragma unroll
        for (int gi = 0; gi < GPS; ++gi) {
          // the group's B operands and scales (x 2^9: a code's byte is q * 2^-9)
          long b[P8_TJ][CPG];
          float s[P8_TJ];
#pragma unroll
          for (int j = 0; j < P8_TJ; ++j) {
#pragma unroll
            for (int ci = 0; ci < CPG; ++ci) {
              const uint32_t w = wr[u][j][gi * CPG + ci];
              b[j][ci] = as_long(w & 0x0F0F0F0Fu, (w >> 4) & 0x0F0F0F0Fu);
            }
            s[j] = __uint_as_float(sr[u][j][gi] << 16) * 512.f;
          }
          // a row tile's sums over the group start from zero and are then added, scaled, to its accumulators; the
          // four column tiles' matrix instructions go out before the first of them is read back
#pragma unroll
          for (int r = 0; r < RT; ++r) {
            long a[CPG];
#pragma unroll
            for (int ci = 0; ci < CPG; ++ci)
              a[ci] = *reinterpret_cast<const long*>(abuf + 16 * r * P8_AROW + (gi * CPG + ci) * 32);
            f32x4_t cur[P8_TJ];
#pragma unroll
            for (int j = 0; j < P8_TJ; ++j)
              cur[j] = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(a[0], b[j][0], (f32x4_t){0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
            if constexpr (CPG == 2) {
#pragma unroll
              for (int j = 0; j < P8_TJ; ++j) cur[j] = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(a[1], b[j][1], cur[j], 0, 0, 0);
            }
#pragma unroll
            for (int j = 0; j < P8_TJ; ++j)
#pragma unroll
              for (int e = 0; e < 4; ++e) acc[j][r][e] = fmaf(cur[j][e], s[j], acc[j][r][e]);
            // (a row tile at a time: left free, the scheduler hoists every tile's LDS reads and partial sums to the
            // head of the group and spills the accumulators)
            __builtin_amdgcn_sched_barrier(0);
          }
        }
        load_w(min(step + 2, last), wr[u], sr[u]);     // wr[u] has just been used for the last time
        store_a(1 - u, ar);
        __syncthreads();
      }
    }
  }

  // bias term: acc += xs (bf16 [M, KG]) . biases (bf16 [KG, npad]) over the groups, 32 a matrix instruction, zeros
  // past KG (qmm_prefill8.cu:186-188)
#pragma unroll 1
  for (int g0 = 0; g0 < KG; g0 += 32) {
    bf16x8_t bb[P8_TJ];
#pragma unroll
    for (int j = 0; j < P8_TJ; ++j) {
      uint32_t v[4];
#pragma unroll
      for (int p = 0; p < 4; ++p) {
        const int g = g0 + 8 * kq + 2 * p;
        const uint32_t lo = g < KG ? B[(size_t)g * npad + (cp[j] >> 1)] : 0u;
        const uint32_t hi = g + 1 < KG ? B[(size_t)(g + 1) * npad + (cp[j] >> 1)] : 0u;
        v[p] = lo | (hi << 16);
      }
      const u32x4_t q = {v[0], v[1], v[2], v[3]};
      bb[j] = __builtin_bit_cast(bf16x8_t, q);
    }
#pragma unroll
    for (int r = 0; r < RT; ++r) {
      const uint16_t* xr = XS + (size_t)(m0 + min(16 * r + c, cnt - 1)) * KG;
      uint32_t v[4];
#pragma unroll
      for (int p = 0; p < 4; ++p) {
        const int g = g0 + 8 * kq + 2 * p;
        const uint32_t lo = g < KG ? xr[g] : 0u;
        const uint32_t hi = g + 1 < KG ? xr[g + 1] : 0u;
        v[p] = lo | (hi << 16);
      }
      const u32x4_t q = {v[0], v[1], v[2], v[3]};
      const bf16x8_t xa = __builtin_bit_cast(bf16x8_t, q);
#pragma unroll
      for (int j = 0; j < P8_TJ; ++j) acc[j][r] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xa, bb[j], acc[j][r], 0, 0, 0);
    }
  }

  // D[row 4 kq + i][column c] of each 16 x 16 tile, times the row's scale
#pragma unroll
  for (int r = 0; r < RT; ++r) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int row = 16 * r + 4 * kq + i;
      if (row >= cnt) continue;
      const float a = A[m0 + row];
      const size_t base = (size_t)(m0 + row) * N;
#pragma unroll
      for (int j = 0; j < P8_TJ; ++j) {
        if (!jok[j]) continue;
        const float v = acc[j][r][i] * a;
        if constexpr (F32) reinterpret_cast<float*>(out)[base + ocol[j]] = v;
        else reinterpret_cast<uint16_t*>(out)[base + ocol[j]] = (uint16_t)f32_bf16_bits(v);
      }
    }
  }
}

template <int GS, bool F32>
__global__ void __launch_bounds__(P8_THREADS, 1)
    qmm_prefill8_kernel(const uint8_t* __restrict__ X8, const uint16_t* __restrict__ XS, const float* __restrict__ A,
                        const uint32_t* __restrict__ W, const uint16_t* __restrict__ S, const uint16_t* __restrict__ B,
                        void* __restrict__ out, int M, int N, int KG, int npad) {
  extern __shared__ __align__(16) unsigned char smem[];
  const int ct = (N + 255) >> 8;
  const int rt = blockIdx.x / ct, cbt = blockIdx.x - rt * ct;
  const int m0 = rt * P8_ROWS, cnt = min(P8_ROWS, M - m0);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, c = lane & 15, kq = lane >> 4;
  const int tiles = npad >> 6, tile = cbt * 4 + (wave >> 1), half = wave & 1;      // a 64-column tile a pair of waves
  const bool ok = tile < tiles;
  const __amdgpu_buffer_rsrc_t codes = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<uint32_t*>(W), 0, (uint32_t)tiles * KG * (GS / 32) * 1024u, 0x00020000);
  const __amdgpu_buffer_rsrc_t scales =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(S), 0, (uint32_t)KG * npad * 2u, 0x00020000);
  uint32_t wp[P8_TJ], cp[P8_TJ];
  int ocol[P8_TJ];
  bool jok[P8_TJ];
#pragma unroll
  for (int j = 0; j < P8_TJ; ++j) {
    const int in_tile = 32 * half + 16 * j + c;
    const int col = (ok ? tile : 0) * 64 + in_tile;                 // columns up to npad are stored zeros
    wp[j] = ((uint32_t)(ok ? tile : 0) * KG * (GS / 32) * 256u + in_tile * 4 + kq) * 4u;
    cp[j] = col * 2;
    ocol[j] = col;
    jok[j] = ok && col < N;
  }
  const int K = KG * GS;
  if (cnt <= 32) prefill8_body<GS, F32, 2>(X8, XS, A, codes, scales, B, out, m0, cnt, N, K, KG, npad, wp, cp, ocol, jok, smem);
  else if (cnt <= 64) prefill8_body<GS, F32, 4>(X8, XS, A, codes, scales, B, out, m0, cnt, N, K, KG, npad, wp, cp, ocol, jok, smem);
  else prefill8_body<GS, F32, 8>(X8, XS, A, codes, scales, B, out, m0, cnt, N, K, KG, npad, wp, cp, ocol, jok, smem);
}

}  // namespace
}  // namespace tf

using namespace tf;

extern "C" int tf_quantize_rows(const uint16_t* x, int64_t ldx, int m, int k, int gs, uint8_t* x8, uint16_t* xs,
                                float* a, tf_stream_t stream) {
  clear_error();
  TF_REQUIRE(gs == 32 || gs == 64, "quantize_rows: groups of 32 or 64 inputs, not %d", gs);
  TF_REQUIRE(x && x8 && xs && a && m >= 1, "quantize_rows: null pointer or empty shape");
  TF_REQUIRE(k >= gs && k % gs == 0 && k % 32 == 0, "quantize_rows takes K a multiple of the group and of 32");
  TF_REQUIRE(aligned16(x) && (m == 1 || ldx % 8 == 0) && aligned16(x8), "quantize_rows: rows must start on 16-byte boundaries");
  if (gs == 64) quantize_rows_kernel<64><<<m, 256, 0, as_stream(stream)>>>(x, ldx, k, x8, xs, a);
  else quantize_rows_kernel<32><<<m, 256, 0, as_stream(stream)>>>(x, ldx, k, x8, xs, a);
  TF_LAUNCH_OK("tf_quantize_rows");
  return 0;
}

extern "C" int tf_qmm_prefill8(const uint8_t* x8, const uint16_t* xs, const float* a, const uint32_t* weight,
                               const uint16_t* scales, const uint16_t* biases, void* out, int m, int n, int k, int gs,
                               int f32, int tile, tf_stream_t stream) {
  clear_error();
  TF_REQUIRE(gs == 32 || gs == 64, "qmm_prefill8: groups of 32 or 64 inputs, not %d", gs);
  TF_REQUIRE(tile >= 0 && tile <= 11, "tile 0-11");
  TF_REQUIRE(x8 && xs && a && weight && scales && biases && out && m >= 1 && n >= 1,
             "qmm_prefill8: null pointer or empty shape");
  TF_REQUIRE(k >= 64 && k % 64 == 0, "qmm_prefill8 takes K in whole steps of 64 inputs, not %d", k);
  TF_REQUIRE(aligned16(x8), "qmm_prefill8: x8 must be 16-byte aligned");
  const int kg = k / gs, npad = (n + 127) / 128 * 128;
  TF_REQUIRE((int64_t)npad * k / 2 < (1ll << 32), "qmm_prefill8: a weight of %d x %d is past the 4 GB a launch addresses", n, k);
  const int64_t grid = (int64_t)((m + P8_ROWS - 1) / P8_ROWS) * ((n + 255) / 256);
  TF_REQUIRE(grid <= 0x7FFFFFFF, "qmm_prefill8: grid too large");
  hipStream_t s = as_stream(stream);
#define TF_GO(GS_, F32_)                                                                                        \
  qmm_prefill8_kernel<GS_, F32_><<<(unsigned)grid, P8_THREADS, 2 * P8_STAGE, s>>>(x8, xs, a, weight, scales, biases, \
                                                                                  out, m, n, kg, npad)
  if (gs == 64) {
    if (f32) TF_GO(64, true); else TF_GO(64, false);
  } else {
    if (f32) TF_GO(32, true); else TF_GO(32, false);
  }
#undef TF_GO
  TF_LAUNCH_OK("tf_qmm_prefill8");
  return 0;
}
