// Fused producers of the quantized matmuls' inputs: residual add (plain, or the MoE layer's weighted pair outputs),
// RMSNorm, and the fp32 group sums of the normed bf16 row that the 4-bit kernels take as `xs` -- one launch, a
// workgroup of 512 threads a row, the row held in registers between the two passes.  A row's bits depend on that row alone.
// (families/qwen3_5/cuda/glue.py:10-41 `add_rmsnorm`, families/nemotron_h/cuda/glue.py:103-141 `add_moe_norm`.)

#include "tf_common.h"

namespace tf {
namespace {

enum { DELTA_NONE = 0, DELTA_BF16 = 1, DELTA_PAIRS_F32 = 2, DELTA_PAIRS_BF16 = 3 };

constexpr int NORM_THREADS = 512, NORM_WAVES = NORM_THREADS / 64;

__device__ __forceinline__ void load4(const void* p, bool is_bf16, size_t at, float (&v)[4]) {
  if (is_bf16) {
    const uint2 u = *reinterpret_cast<const uint2*>(static_cast<const uint16_t*>(p) + at);
    v[0] = bf16_lo(u.x);
    v[1] = bf16_hi(u.x);
    v[2] = bf16_lo(u.y);
    v[3] = bf16_hi(u.y);
  } else {
    const f32x4_t f = *reinterpret_cast<const f32x4_t*>(static_cast<const float*>(p) + at);
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] = f[e];
  }
}

__device__ __forceinline__ void store4(uint16_t* p, size_t at, const float (&v)[4]) {
  *reinterpret_cast<uint2*>(p + at) = make_uint2(pack_bf16(v[0], v[1]), pack_bf16(v[2], v[3]));
}

// NI: runs of four columns a thread (thread t holds columns 4 (t + 512 i) .. + 3 for i < NI), so D <= 2048 NI.
// The group of GS columns is GS / 4 neighbouring threads of one i: its sum is a butterfly over those lanes.
// The pair outputs of KB slots and all NI runs are requested together: one trip to memory a batch of slots.
template <int NI, int GS>
__global__ void __launch_bounds__(NORM_THREADS)
    add_norm_kernel(const uint16_t* __restrict__ X, const void* __restrict__ delta, int kind,
                    const float* __restrict__ Wt, int S, int NR, const uint16_t* __restrict__ W, float eps,
                    uint16_t* __restrict__ H, uint16_t* __restrict__ Y, float* __restrict__ XS, int D) {
  constexpr int KB = NI == 1 ? 8 : NI == 2 ? 4 : 2;
  __shared__ float part[NORM_WAVES];
  const int row = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  float v[NI][4], wn[NI][4];
#pragma unroll
  for (int i = 0; i < NI; ++i) {
    const int d = 4 * (tid + NORM_THREADS * i);
#pragma unroll
    for (int e = 0; e < 4; ++e) v[i][e] = wn[i][e] = 0.f;
    if (d >= D) continue;
    load4(X, true, (size_t)row * D + d, v[i]);
    load4(W, true, d, wn[i]);
  }
  if (kind == DELTA_BF16) {
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      const int d = 4 * (tid + NORM_THREADS * i);
      if (d >= D) continue;
      float r[4];
      load4(delta, true, (size_t)row * D + d, r);
#pragma unroll
      for (int e = 0; e < 4; ++e) v[i][e] = round_bf16(v[i][e] + r[e]);
    }
  } else if (kind != DELTA_NONE) {
    // routed = sum over the first NR slots of wt * y, product and sum each rounded to fp32, in slot order; shared =
    // the plain sum of the rest; delta = bf16(routed + shared)
    float ro[NI][4], sh[NI][4];
#pragma unroll
    for (int i = 0; i < NI; ++i)
#pragma unroll
      for (int e = 0; e < 4; ++e) ro[i][e] = sh[i][e] = 0.f;
    for (int k0 = 0; k0 < S; k0 += KB) {
      float w[KB], y[KB][NI][4];
#pragma unroll
      for (int j = 0; j < KB; ++j) {
        const int k = k0 + j < S ? k0 + j : S - 1;
        w[j] = Wt[(size_t)row * S + k];
#pragma unroll
        for (int i = 0; i < NI; ++i) {
          const int d = 4 * (tid + NORM_THREADS * i);
#pragma unroll
          for (int e = 0; e < 4; ++e) y[j][i][e] = 0.f;
          if (d < D) load4(delta, kind == DELTA_PAIRS_BF16, ((size_t)row * S + k) * D + d, y[j][i]);
        }
      }
#pragma unroll
      for (int j = 0; j < KB; ++j) {
        const int k = k0 + j;
        if (k >= S) break;
#pragma unroll
        for (int i = 0; i < NI; ++i)
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            if (k < NR) ro[i][e] = __fadd_rn(ro[i][e], __fmul_rn(w[j], y[j][i][e]));
            else sh[i][e] = __fadd_rn(sh[i][e], y[j][i][e]);
          }
      }
    }
#pragma unroll
    for (int i = 0; i < NI; ++i)
#pragma unroll
      for (int e = 0; e < 4; ++e) v[i][e] = round_bf16(v[i][e] + round_bf16(ro[i][e] + sh[i][e]));
  }
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < NI; ++i) {
    const int d = 4 * (tid + NORM_THREADS * i);
    if (d >= D) continue;
    if (kind != DELTA_NONE) store4(H, (size_t)row * D + d, v[i]);
#pragma unroll
    for (int e = 0; e < 4; ++e) ss = fmaf(v[i][e], v[i][e], ss);
  }
  // sum of squares: lanes by butterfly, then the waves in order
#pragma unroll
  for (int m = 1; m < 64; m <<= 1) ss += __shfl_xor(ss, m);
  if (lane == 0) part[wave] = ss;
  __syncthreads();
  float total = part[0];
#pragma unroll
  for (int q = 1; q < NORM_WAVES; ++q) total += part[q];
  const float inv = 1.0f / sqrtf(total / (float)D + eps);
#pragma unroll
  for (int i = 0; i < NI; ++i) {
    const int d = 4 * (tid + NORM_THREADS * i);
    float o[4] = {0.f, 0.f, 0.f, 0.f};
    if (d < D) {
#pragma unroll
      for (int e = 0; e < 4; ++e) o[e] = round_bf16(__fmul_rn(__fmul_rn(v[i][e], inv), wn[i][e]));
      store4(Y, (size_t)row * D + d, o);
    }
    // D is whole groups, so a group is all inside or all outside the row; the threads of one i are whole groups
    float g = (o[0] + o[1]) + (o[2] + o[3]);
#pragma unroll
    for (int m = 1; m < GS / 4; m <<= 1) g += __shfl_xor(g, m);
    if (d < D && (lane & (GS / 4 - 1)) == 0) XS[(size_t)row * (D / GS) + d / GS] = g;
  }
}

template <int GS>
int launch_add_norm(const uint16_t* x, const void* delta, int kind, const float* wts, int slots, int routed,
                    const uint16_t* w, float eps, uint16_t* h, uint16_t* y, float* xs, int rows, int d, hipStream_t s) {
#define TF_AN(NI_)                                                                                                   \
  if (d <= 2048 * NI_) {                                                                                             \
    add_norm_kernel<NI_, GS><<<rows, NORM_THREADS, 0, s>>>(x, delta, kind, wts, slots, routed, w, eps, h, y, xs, d); \
    TF_LAUNCH_OK("tf_add_norm");                                                                                     \
    return 0;                                                                                                        \
  }
  TF_AN(1) TF_AN(2) TF_AN(4) TF_AN(8)
#undef TF_AN
  set_error("add_norm: rows of at most 16384 values, not %d", d);
  return 1;
}

}  // namespace
}  // namespace tf

using namespace tf;

extern "C" int tf_add_norm(const uint16_t* x, const void* delta, int delta_kind, const float* wts, int slots, int routed,
                           const uint16_t* w, float eps, uint16_t* h, uint16_t* y, float* xs, int rows, int d, int gs,
                           tf_stream_t stream) {
  clear_error();
  TF_REQUIRE(x && w && y && xs, "add_norm: null pointer argument");
  TF_REQUIRE(delta_kind >= DELTA_NONE && delta_kind <= DELTA_PAIRS_BF16, "add_norm: delta kind 0-3, not %d", delta_kind);
  TF_REQUIRE(delta_kind == DELTA_NONE || (delta && h), "add_norm: a delta needs its tensor and h");
  TF_REQUIRE(delta_kind < DELTA_PAIRS_F32 || (wts && slots >= 1 && routed >= 0 && routed <= slots),
             "add_norm: pair outputs need wts [rows, slots] and 0 <= routed <= slots");
  TF_REQUIRE(rows >= 1 && d >= gs && (gs == 32 || gs == 64 || gs == 128) && d % gs == 0,
             "add_norm: rows of whole groups of 32, 64 or 128 values");
  TF_REQUIRE((((uintptr_t)x | (uintptr_t)y | (uintptr_t)w | (uintptr_t)h | (uintptr_t)delta) & 7) == 0,
             "add_norm: tensors must be 8-byte aligned");
  hipStream_t s = as_stream(stream);
  if (gs == 32) return launch_add_norm<32>(x, delta, delta_kind, wts, slots, routed, w, eps, h, y, xs, rows, d, s);
  if (gs == 64) return launch_add_norm<64>(x, delta, delta_kind, wts, slots, routed, w, eps, h, y, xs, rows, d, s);
  return launch_add_norm<128>(x, delta, delta_kind, wts, slots, routed, w, eps, h, y, xs, rows, d, s);
}
