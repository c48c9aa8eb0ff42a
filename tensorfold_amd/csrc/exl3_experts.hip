// EXL3 routed experts, any codebook and a width per expert: tf_exl3x_rot_in, tf_exl3x_grouped,
// tf_exl3x_gateup_epilogue, tf_exl3x_down_combine  (reference: cuda/exl3/experts.py:173-202, experts.cu,
// experts_grouped.cuh).
//
// Pairs p = row * slots + slot whose pick is a routed expert (0 <= pick < E) are grouped by expert into items of at
// most 16 (tf_experts_plan); an item is one 16-row MFMA pass of the dense linear's wave walk over the expert's own
// trellis at the expert's own width, its rows gathered through `members`.  K splits write fp32 partials that the
// epilogues add in split order; every butterfly and sum runs in a fixed order and no row reads another row, so a
// row's bits do not depend on the window it arrives in.
//
// tf_exl3x_plan_rot_in puts the grouping and the input rotation into one launch (workgroup 0 groups, the others
// rotate; neither needs the other's result).

#include "exl3_decode.h"
#include "routing.h"

namespace tf {
namespace {

constexpr int XWK = 4;          // waves a workgroup of the grouped kernel

// xg[p] = fp16(((x[row] * suh_g[e]) H) / sqrt(128)) and the same with suh_u into xu[p], a wave a (pair, block of 128)
__global__ void __launch_bounds__(256)
    x_rot_in_kernel(const void* __restrict__ x, int x_dtype, int64_t x_stride, const int* __restrict__ pick,
                    const uint16_t* __restrict__ suh0, const uint16_t* __restrict__ suh1, uint16_t* __restrict__ out0,
                    uint16_t* __restrict__ out1, int K, int slots, int E) {
  const int blk = blockIdx.x * 4 + (threadIdx.x >> 6), p = blockIdx.y, mat = blockIdx.z, lane = threadIdx.x & 63;
  if (blk * 128 >= K) return;
  const int e = pick[p];
  if (e < 0 || e >= E) return;
  const int k = blk * 128 + 2 * lane;
  float a, b, sa, sb;
  load2(x, x_dtype, (size_t)(p / slots) * x_stride + k, a, b);
  load2(mat ? suh1 : suh0, TF_F16, (size_t)e * K + k, sa, sb);
  a *= sa;
  b *= sb;
  fwht128(a, b, lane);
  store2(mat ? out1 : out0, TF_F16, (size_t)p * K + k, a * HAD_SCALE, b * HAD_SCALE);
}

// The grouping and the input rotation in one launch: workgroup 0 makes the plan (tf_experts_plan's, up to 1,024
// pairs), every other workgroup rotates sixteen (matrix, pair, block of 128) units as x_rot_in_kernel does.
__global__ void __launch_bounds__(PLAN_THREADS)
    plan_rot_in_kernel(const void* __restrict__ x, int x_dtype, int64_t x_stride, const int* __restrict__ pick,
                       const uint16_t* __restrict__ suh0, const uint16_t* __restrict__ suh1,
                       uint16_t* __restrict__ out0, uint16_t* __restrict__ out1, int K, int slots, int E, int P, int T,
                       int* __restrict__ members, int* __restrict__ items, int* __restrict__ counts) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  if (blockIdx.x == 0) {
    __shared__ int pk[PLAN_THREADS];
    __shared__ PlanLds plan;
    plan_small(pick, P, E, T, members, items, counts, pk, plan);
    return;
  }
  const int KB = K / 128, unit = (blockIdx.x - 1) * (PLAN_THREADS / 64) + wave;
  const int mats = suh1 ? 2 : 1;
  if (unit >= P * KB * mats) return;
  const int mat = unit / (P * KB), rest = unit - mat * (P * KB), p = rest / KB, blk = rest - p * KB;
  const int e = pick[p];
  if (e < 0 || e >= E) return;
  const int k = blk * 128 + 2 * lane;
  float a, b, sa, sb;
  load2(x, x_dtype, (size_t)(p / slots) * x_stride + k, a, b);
  load2(mat ? suh1 : suh0, TF_F16, (size_t)e * K + k, sa, sb);
  a *= sa;
  b *= sb;
  fwht128(a, b, lane);
  store2(mat ? out1 : out0, TF_F16, (size_t)p * K + k, a * HAD_SCALE, b * HAD_SCALE);
}

struct GroupedArgs {
  const uint16_t* x[2];        // rotated inputs fp16 [P, K] of matrix 0 and 1
  const int64_t* tp[2];        // each expert's trellis address
  const int* k2[2];            // each expert's half-bits a value
  const int* items;            // (expert, first member, count <= 16) rows
  const int* counts;           // counts[0] = items
  const int* members;          // pairs ordered by expert
  float* Z;                    // [mats * SK, P, N] partial sums
  int mats, K, N, P, SK, E;
};

// the sum over K splits, in split order, of the two columns of pair p that lane holds
__device__ __forceinline__ float2 split_sum(const float* z, size_t split_stride, int SK) {
  float2 s = {0.f, 0.f};
  for (int q0 = 0; q0 < SK; q0 += 8) {
    float2 v[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = *reinterpret_cast<const float2*>(z + (size_t)(q0 + j < SK ? q0 + j : SK - 1) * split_stride);
#pragma unroll
    for (int j = 0; j < 8; ++j)
      if (q0 + j < SK) {
        s.x += v[j].x;
        s.y += v[j].y;
      }
  }
  return s;
}

__device__ __forceinline__ float half_f32(uint16_t v) { return __half2float(__ushort_as_half(v)); }

// Pair p's block of 128 of the width after gate and up (a wave; n = the lane's first column): splits summed, rotated,
// * svh, SwiGLU (act_mode 0: bf16 roundings; 1: fp32), then xd = fp16(((act * suh_d) H) / sqrt(128))
__device__ __forceinline__ void gateup_row(const float* __restrict__ Z, int p, int e, int n, int lane,
                                           const uint16_t* __restrict__ svh_g, const uint16_t* __restrict__ svh_u,
                                           const uint16_t* __restrict__ suh_d, uint16_t* __restrict__ xd, int P, int N,
                                           int SK, float limit, int act_mode) {
  const size_t ss = (size_t)P * N;
  float2 gv = split_sum(Z + (size_t)p * N + n, ss, SK);
  float2 uv = split_sum(Z + (size_t)SK * ss + (size_t)p * N + n, ss, SK);
  fwht128(gv.x, gv.y, lane);
  fwht128(uv.x, uv.y, lane);
  const uint32_t sg = *reinterpret_cast<const uint32_t*>(svh_g + (size_t)e * N + n);
  const uint32_t su = *reinterpret_cast<const uint32_t*>(svh_u + (size_t)e * N + n);
  const uint32_t sd = *reinterpret_cast<const uint32_t*>(suh_d + (size_t)e * N + n);
  const float g2[2] = {gv.x, gv.y}, u2[2] = {uv.x, uv.y};
  float v[2];
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const float wg = half_f32((uint16_t)(sg >> (16 * j))), wu = half_f32((uint16_t)(su >> (16 * j)));
    float act;
    if (act_mode == 0) {
      const float gg = fminf(round_bf16(g2[j] * HAD_SCALE * wg), limit);
      const float uu = fminf(fmaxf(round_bf16(u2[j] * HAD_SCALE * wu), -limit), limit);
      act = round_bf16(round_bf16(gg / (1.f + expf(-gg))) * uu);
    } else {
      const float gg = fminf(g2[j] * HAD_SCALE * wg, limit);
      const float uu = fminf(fmaxf(u2[j] * HAD_SCALE * wu, -limit), limit);
      act = gg / (1.f + expf(-gg)) * uu;
    }
    v[j] = act * half_f32((uint16_t)(sd >> (16 * j)));
  }
  fwht128(v[0], v[1], lane);
  store2(xd, TF_F16, (size_t)p * N + n, v[0] * HAD_SCALE, v[1] * HAD_SCALE);
}

// Pair p's block of 128 of the output after down (a wave): ((splits summed) H / sqrt(128)) * svh_d
__device__ __forceinline__ float2 down_row(const float* __restrict__ Z, int p, int e, int n, int lane,
                                           const uint16_t* __restrict__ svh_d, int P, int D, int SK) {
  float2 v = split_sum(Z + (size_t)p * D + n, (size_t)P * D, SK);
  fwht128(v.x, v.y, lane);
  const uint32_t sv = *reinterpret_cast<const uint32_t*>(svh_d + (size_t)e * D + n);
  return make_float2(v.x * HAD_SCALE * half_f32((uint16_t)sv), v.y * HAD_SCALE * half_f32((uint16_t)(sv >> 16)));
}

// One item, one 128-column block, one K split, one matrix: the dense linear's pass with gathered rows.
template <int K2, int CB>
__device__ __forceinline__ void grouped_body(const GroupedArgs& g, const uint32_t* T, const uint16_t* xh, int first,
                                             int cnt, int mat, float* red) {
  constexpr int TW = tile_words<K2>();
  const int nb = blockIdx.x, split = blockIdx.y;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, c = lane & 15, kq = lane >> 4;
  const int L = 4 * (c & 7) + kq, h = c >> 3;
  const int pairs = g.K >> 5, slot = split * XWK + wave, nslots = g.SK * XWK;
  const int pr0 = (int)((long long)slot * pairs / nslots), pr1 = (int)((long long)(slot + 1) * pairs / nslots);
  const int64_t stride_k = (int64_t)(g.N >> 4) * TW;          // the checkpoint's order: [K / 16][N / 16][TW] words
  const uint32_t* tiles = T + (size_t)nb * 8 * TW;
  f32x4_t acc[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) acc[j] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
  // the A operand's row: lane (row c, quarter kq); rows past the item read its last row and are dropped
  const int pc = g.members[first + (c < cnt ? c : cnt - 1)];
  const uint16_t* xr = xh + (size_t)pc * g.K + 2 * kq;
  uint32_t* stage = reinterpret_cast<uint32_t*>(red) + wave * (16 * 128);
  wave_block<K2, CB>(xr, tiles, stride_k, pr0, pr1, stage, lane, L, h, acc);
  // D[row 4 kq + i][column c] of column tile j -> red[wave][row][16 j + c]
  __syncthreads();
#pragma unroll
  for (int j = 0; j < 8; ++j)
#pragma unroll
    for (int i = 0; i < 4; ++i) red[(wave * 16 + 4 * kq + i) * 128 + 16 * j + c] = acc[j][i];
  __syncthreads();
  // a wave a row: the waves' sums in wave order, two columns a lane
  float* zs = g.Z + (size_t)(mat * g.SK + split) * g.P * g.N + nb * 128 + 2 * lane;
  for (int r = wave; r < cnt; r += XWK) {
    float2 s = *reinterpret_cast<const float2*>(red + r * 128 + 2 * lane);
    for (int w = 1; w < XWK; ++w) {
      const float2 q = *reinterpret_cast<const float2*>(red + (w * 16 + r) * 128 + 2 * lane);
      s.x += q.x;
      s.y += q.y;
    }
    *reinterpret_cast<float2*>(zs + (size_t)g.members[first + r] * g.N) = s;
  }
}

// grid (N / 128, SK, max items * mats); the width is the expert's own
template <int CB>
__global__ void __launch_bounds__(XWK * 64) grouped_kernel(const GroupedArgs g) {
  extern __shared__ __align__(16) float red[];              // [XWK][16][128]
  const int it = blockIdx.z / g.mats, mat = blockIdx.z - it * g.mats;
  if (it >= g.counts[0]) return;
  const int e = g.items[3 * it];
  if (e < 0 || e >= g.E) return;                            // an id past the routed experts (a shared slot): not ours
  const int first = g.items[3 * it + 1], cnt = g.items[3 * it + 2];
  const uint32_t* T = reinterpret_cast<const uint32_t*>(g.tp[mat][e]);
  const uint16_t* xh = g.x[mat];
  switch (g.k2[mat][e]) {
#define TF_CASE(K2_) \
  case K2_:          \
    grouped_body<K2_, CB>(g, T, xh, first, cnt, mat, red); \
    break;
    TF_CASE(2) TF_CASE(3) TF_CASE(4) TF_CASE(5) TF_CASE(6) TF_CASE(7) TF_CASE(8) TF_CASE(9) TF_CASE(10) TF_CASE(11)
    TF_CASE(12) TF_CASE(13) TF_CASE(14) TF_CASE(15) TF_CASE(16)
#undef TF_CASE
    default: break;                                         // widths are checked on the host
  }
}


// a wave a (pair, block of 128 of the width): splits summed, rotated, * svh, SwiGLU (act_mode 0: bf16 roundings;
// 1: fp32), then xd = fp16(((act * suh_d) H) / sqrt(128))
__global__ void __launch_bounds__(256)
    gateup_epilogue_kernel(const float* __restrict__ Z, const int* __restrict__ pick, const uint16_t* __restrict__ svh_g,
                           const uint16_t* __restrict__ svh_u, const uint16_t* __restrict__ suh_d,
                           uint16_t* __restrict__ xd, int P, int N, int SK, int E, float limit, int act_mode) {
  const int blk = blockIdx.x * 4 + (threadIdx.x >> 6), p = blockIdx.y, lane = threadIdx.x & 63;
  if (blk * 128 >= N) return;
  const int e = pick[p];
  if (e < 0 || e >= E) return;
  gateup_row(Z, p, e, blk * 128 + 2 * lane, lane, svh_g, svh_u, suh_d, xd, P, N, SK, limit, act_mode);
}

// grid (D / 128, rows): y[p] = ((splits summed) H / sqrt(128)) * svh_d for the routed slots (the others keep what
// the caller put in y), a wave a slot; then out[r] = the fma chain over the slots in order of wts * y, fp32
__global__ void __launch_bounds__(256)
    down_combine_kernel(const float* __restrict__ Z, const int* __restrict__ pick, const uint16_t* __restrict__ svh_d,
                        float* __restrict__ y, const float* __restrict__ wts, float* __restrict__ out, int P, int D, int SK,
                        int E, int slots) {
  extern __shared__ __align__(16) float part[];             // [slots][128]
  const int blk = blockIdx.x, r = blockIdx.y, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int n = blk * 128 + 2 * lane;
  for (int k = wave; k < slots; k += 4) {
    const int p = r * slots + k;
    const int e = pick[p];
    float2 o;
    if (e >= 0 && e < E) {
      o = down_row(Z, p, e, n, lane, svh_d, P, D, SK);
      *reinterpret_cast<float2*>(y + (size_t)p * D + n) = o;
    } else if (wts) {
      o = *reinterpret_cast<const float2*>(y + (size_t)p * D + n);
    }
    if (wts) *reinterpret_cast<float2*>(part + k * 128 + 2 * lane) = o;
  }
  if (!wts) return;
  __syncthreads();
  if (wave) return;
  float a0 = 0.f, a1 = 0.f;
  for (int q = 0; q < slots; ++q) {
    const float w = wts[(size_t)r * slots + q];
    const float2 u = *reinterpret_cast<const float2*>(part + q * 128 + 2 * lane);
    a0 = fmaf(w, u.x, a0);
    a1 = fmaf(w, u.y, a1);
  }
  *reinterpret_cast<float2*>(out + (size_t)r * D + n) = make_float2(a0, a1);
}

}  // namespace
}  // namespace tf

using namespace tf;

extern "C" int tf_exl3x_rot_in(const void* x, int x_dtype, int64_t x_stride, const int32_t* pick, const uint16_t* suh0,
                               const uint16_t* suh1, uint16_t* out0, uint16_t* out1, int rows, int slots, int k,
                               int experts, tf_stream_t stream) {
  clear_error();
  TF_REQUIRE(x && pick && suh0 && out0 && (!suh1 == !out1), "exl3x rot_in: null pointer argument");
  TF_REQUIRE(x_dtype == TF_F16 || x_dtype == TF_BF16 || x_dtype == TF_F32, "x: expected fp16, bf16 or fp32");
  TF_REQUIRE(rows >= 1 && slots >= 1 && (int64_t)rows * slots <= 65535, "exl3x rot_in: 1 to 65535 pairs");
  TF_REQUIRE(k >= 128 && k % 128 == 0 && x_stride >= k && x_stride % 2 == 0, "x rows of K values, K a multiple of 128");
  TF_REQUIRE(((uintptr_t)x & 7) == 0 && aligned16(out0) && aligned16(out1), "x 8-byte, outputs 16-byte aligned");
  const dim3 grid((k / 128 + 3) / 4, rows * slots, suh1 ? 2 : 1);
  x_rot_in_kernel<<<grid, 256, 0, as_stream(stream)>>>(x, x_dtype, x_stride, pick, suh0, suh1, out0, out1, k, slots, experts);
  TF_LAUNCH_OK("tf_exl3x_rot_in");
  return 0;
}

extern "C" int tf_exl3x_grouped(const uint16_t* x0, const uint16_t* x1, const int64_t* tp0, const int64_t* tp1,
                                const int32_t* k2_0, const int32_t* k2_1, const int32_t* items, const int32_t* counts,
                                const int32_t* members, float* z, int mats, int k, int n, int pairs, int sk, int cb,
                                int experts, int max_items, tf_stream_t stream) {
  clear_error();
  TF_REQUIRE(x0 && tp0 && k2_0 && items && counts && members && z, "exl3x grouped: null pointer argument");
  TF_REQUIRE(mats == 1 || (mats == 2 && x1 && tp1 && k2_1), "exl3x grouped: one matrix, or two with their tables");
  TF_REQUIRE(k >= 128 && n >= 128 && k % 128 == 0 && n % 128 == 0, "K and N must be multiples of 128");
  TF_REQUIRE(sk >= 1 && sk <= 64 && (int64_t)sk * XWK <= k / 32, "K / 32 = %d tile pairs do not split over %d x %d waves",
             k / 32, sk, XWK);
  TF_REQUIRE(pairs >= 1 && experts >= 1 && max_items >= 1 && (int64_t)max_items * mats <= 65535,
             "exl3x grouped: 1 to 65535 item launches");
  TF_REQUIRE(aligned16(x0) && aligned16(x1) && ((uintptr_t)z & 7) == 0, "inputs 16-byte, Z 8-byte aligned");
  GroupedArgs g;
  g.x[0] = x0, g.x[1] = mats == 2 ? x1 : x0;
  g.tp[0] = tp0, g.tp[1] = mats == 2 ? tp1 : tp0;
  g.k2[0] = k2_0, g.k2[1] = mats == 2 ? k2_1 : k2_0;
  g.items = items, g.counts = counts, g.members = members, g.Z = z;
  g.mats = mats, g.K = k, g.N = n, g.P = pairs, g.SK = sk, g.E = experts;
  const dim3 grid((unsigned)(n / 128), (unsigned)sk, (unsigned)(max_items * mats));
  const size_t smem = (size_t)XWK * 16 * 128 * sizeof(float);
  hipStream_t s = as_stream(stream);
  if (cb == 0) grouped_kernel<0><<<grid, XWK * 64, smem, s>>>(g);
  else if (cb == 1) grouped_kernel<1><<<grid, XWK * 64, smem, s>>>(g);
  else if (cb == 2) grouped_kernel<2><<<grid, XWK * 64, smem, s>>>(g);
  else {
    set_error("exl3x grouped: codebook 0, 1 or 2, not %d", cb);
    return 1;
  }
  TF_LAUNCH_OK("tf_exl3x_grouped");
  return 0;
}

extern "C" int tf_exl3x_plan_rot_in(const void* x, int x_dtype, int64_t x_stride, const int32_t* pick,
                                    const uint16_t* suh0, const uint16_t* suh1, uint16_t* out0, uint16_t* out1, int rows,
                                    int slots, int k, int experts, int tile, int32_t* members, int32_t* items,
                                    int32_t* counts, tf_stream_t stream) {
  clear_error();
  TF_REQUIRE(x && pick && suh0 && out0 && (!suh1 == !out1) && members && items && counts,
             "exl3x plan_rot_in: null pointer argument");
  TF_REQUIRE(x_dtype == TF_F16 || x_dtype == TF_BF16 || x_dtype == TF_F32, "x: expected fp16, bf16 or fp32");
  TF_REQUIRE(rows >= 1 && slots >= 1 && (int64_t)rows * slots <= PLAN_THREADS, "exl3x plan_rot_in: at most %d pairs",
             PLAN_THREADS);
  TF_REQUIRE(experts >= 1 && experts <= EMAX, "experts: at most %d experts", EMAX);
  TF_REQUIRE(tile == 16, "exl3x plan_rot_in: items hold 16 pairs");
  TF_REQUIRE(k >= 128 && k % 128 == 0 && x_stride >= k && x_stride % 2 == 0, "x rows of K values, K a multiple of 128");
  TF_REQUIRE(((uintptr_t)x & 7) == 0 && aligned16(out0) && aligned16(out1), "x 8-byte, outputs 16-byte aligned");
  const int64_t units = (int64_t)rows * slots * (k / 128) * (suh1 ? 2 : 1);
  const int per = PLAN_THREADS / 64;
  plan_rot_in_kernel<<<dim3((unsigned)(1 + (units + per - 1) / per)), PLAN_THREADS, 0, as_stream(stream)>>>(
      x, x_dtype, x_stride, pick, suh0, suh1, out0, out1, k, slots, experts, rows * slots, tile, members, items, counts);
  TF_LAUNCH_OK("tf_exl3x_plan_rot_in");
  return 0;
}

extern "C" int tf_exl3x_gateup_epilogue(const float* z, const int32_t* pick, const uint16_t* svh_g, const uint16_t* svh_u,
                                        const uint16_t* suh_d, uint16_t* xd, int pairs, int n, int sk, int experts,
                                        float limit, int act_mode, tf_stream_t stream) {
  clear_error();
  TF_REQUIRE(z && pick && svh_g && svh_u && suh_d && xd, "exl3x gateup_epilogue: null pointer argument");
  TF_REQUIRE(pairs >= 1 && pairs <= 65535 && n >= 128 && n % 128 == 0 && sk >= 1, "pairs of N values, N a multiple of 128");
  TF_REQUIRE(act_mode == 0 || act_mode == 1, "act_mode 0 (bf16 roundings) or 1 (fp32)");
  const dim3 grid((n / 128 + 3) / 4, pairs);
  gateup_epilogue_kernel<<<grid, 256, 0, as_stream(stream)>>>(z, pick, svh_g, svh_u, suh_d, xd, pairs, n, sk, experts, limit,
                                                              act_mode);
  TF_LAUNCH_OK("tf_exl3x_gateup_epilogue");
  return 0;
}

extern "C" int tf_exl3x_down_combine(const float* z, const int32_t* pick, const uint16_t* svh_d, float* y, const float* wts,
                                     float* out, int rows, int slots, int d, int sk, int experts, tf_stream_t stream) {
  clear_error();
  TF_REQUIRE(z && pick && svh_d && y && (!wts == !out), "exl3x down_combine: null pointer argument");
  TF_REQUIRE(rows >= 1 && rows <= 65535 && slots >= 1 && slots <= 96 && d >= 128 && d % 128 == 0 && sk >= 1,
             "rows of up to 96 slots of D values, D a multiple of 128");
  const dim3 grid(d / 128, rows);
  down_combine_kernel<<<grid, 256, (size_t)slots * 128 * sizeof(float), as_stream(stream)>>>(
      z, pick, svh_d, y, wts, out, rows * slots, d, sk, experts, slots);
  TF_LAUNCH_OK("tf_exl3x_down_combine");
  return 0;
}
