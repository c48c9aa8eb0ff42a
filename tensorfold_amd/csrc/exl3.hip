// EXL3 trellis-coded linear layers: tf_exl3_rot_in, tf_exl3_linear (and their stacked forms), tf_exl3_gate_up,
// tf_exl3_swiglu_rot_in, tf_exl3_unpack, tf_exl3_unpack_k8, tf_exl3_gemm.
//
// The decode primitives are in exl3_decode.h.

#include "exl3_decode.h"

namespace tf {
namespace {

// xh = fp16(((x * suh) H) / sqrt(128)), a wave a (row, block of 128); a workgroup walks rows blockIdx.y, + gridDim.y, ...
// blockIdx.z is the layer of a stack: its own suh [K] and xh [M, K] over the one x.
__global__ void __launch_bounds__(256)
    rot_in_kernel(const void* __restrict__ x, int x_dtype, const uint16_t* __restrict__ suh, uint16_t* __restrict__ xh,
                  int M, int K) {
  const int blk = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (blk * 128 >= K) return;
  suh += (size_t)blockIdx.z * K;
  xh += (size_t)blockIdx.z * M * K;
  const int k = blk * 128 + 2 * lane;
  float sa, sb;
  load2(suh, TF_F16, k, sa, sb);
  // four rows' loads are in flight together
  for (int row0 = blockIdx.y; row0 < M; row0 += 4 * gridDim.y) {
    float a[4], b[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int row = row0 + u * gridDim.y;
      if (row < M) load2(x, x_dtype, (size_t)row * K + k, a[u], b[u]);
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int row = row0 + u * gridDim.y;
      if (row < M) {
        a[u] *= sa;
        b[u] *= sb;
        fwht128(a[u], b[u], lane);
        store2(xh, TF_F16, (size_t)row * K + k, a[u] * HAD_SCALE, b[u] * HAD_SCALE);
      }
    }
  }
}

// The SwiGLU of a stack's two outputs (gate y[0], up y[1], each [M, N]) and the next layer's input rotation in a
// launch of its own: what the linear kernel's workgroups do themselves when they are given xh_next.  A wave a
// (row, block of 128).
__global__ void __launch_bounds__(256)
    swiglu_rot_in_kernel(const void* __restrict__ y, int y_dtype, const uint16_t* __restrict__ suh,
                         uint16_t* __restrict__ xh, int M, int N) {
  const int blk = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (blk * 128 >= N) return;
  const int col = blk * 128 + 2 * lane;
  float sa, sb;
  load2(suh, TF_F16, col, sa, sb);
  for (int row = blockIdx.y; row < M; row += gridDim.y) {
    const size_t at = (size_t)row * N + col;
    float g0, g1, u0, u1;
    load2(y, y_dtype, at, g0, g1);
    load2(y, y_dtype, (size_t)M * N + at, u0, u1);
    swiglu_rot(g0, g1, u0, u1, y_dtype, lane, sa, sb, xh, at);
  }
}

// grid (N / 128, SK, layers); WK waves a block; each wave walks its range of k-tile pairs over the block's eight column
// tiles.  The layers of a stack share K, N, width and codebook; layer z has its own xh [M, K], trellis (stride_layer
// words on), svh and bias [N], y [M, N], Z [SK, M, N] and counters.
// (The second launch bound, waves a SIMD, keeps the kernel within 128 registers at the widths where that costs no
// spill; the widest decodes need a few more and run three waves a SIMD.)
template <int K2, int CB, int WK>
__global__ void __launch_bounds__(WK * 64, K2 <= 12 ? 4 : 1)
    linear_kernel(const uint16_t* __restrict__ xh, const uint32_t* __restrict__ T, int64_t stride_k, int64_t stride_nb,
                  int64_t stride_layer, const uint16_t* __restrict__ svh, const uint16_t* __restrict__ bias,
                  void* __restrict__ y, int y_dtype, float* __restrict__ Z, int* __restrict__ counters, int M, int K,
                  int N, int SK, const uint16_t* __restrict__ suh_next, uint16_t* __restrict__ xh_next) {
  constexpr int TW = tile_words<K2>();
  extern __shared__ __align__(16) float red[];              // [WK][16][128]
  __shared__ int last;
  const int nb = blockIdx.x, split = blockIdx.y, NB = gridDim.x;
  // With xh_next the two layers are an MLP's gate and up: the workgroup that completes a column block over BOTH
  // layers' K splits (one counter for the two, the first layer's) finishes both layers' rows, and writes the next
  // layer's rotated input from their SwiGLU.  y may then be null.
  const bool mlp = xh_next != nullptr;
  const uint16_t *svh0 = svh, *bias0 = bias;
  void* y0 = y;
  float* Z0 = Z;
  if (const size_t z = blockIdx.z) {
    xh += z * M * K;
    T += z * stride_layer;
    svh += z * N;
    if (bias) bias += z * N;
    if (y) y = static_cast<char*>(y) + z * M * N * (y_dtype == TF_F32 ? 4 : 2);
    if (Z) Z += z * SK * M * N;
    if (counters && !mlp) counters += z * 8 * NB * TF_EXL3_COUNTER_STRIDE;
  }
  const int arrivals = mlp ? 2 * SK : SK;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, c = lane & 15, kq = lane >> 4;
  const int L = 4 * (c & 7) + kq, h = c >> 3;
  const int pairs = K >> 5, slot = split * WK + wave, nslots = SK * WK;
  const int pr0 = (int)((long long)slot * pairs / nslots), pr1 = (int)((long long)(slot + 1) * pairs / nslots);
  const uint32_t* tiles = T + (size_t)nb * stride_nb;
  const int col0 = nb * 128;
  TF_MARK(0);

  for (int m0 = 0, pass = 0; m0 < M; m0 += 16, ++pass) {
    const int R = min(16, M - m0);
    f32x4_t acc[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[j] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
    // the A operand's row: lane (row c, quarter kq); rows past the pass read a valid row and are dropped later
    const uint16_t* xr = xh + (size_t)(m0 + (c < R ? c : R - 1)) * K + 2 * kq;
    uint32_t* stage = reinterpret_cast<uint32_t*>(red) + wave * (16 * 128);       // 16 tiles of TW + 2 words
    if (pass) __syncthreads();                 // the previous pass is done with red
    TF_MARK(1);
    wave_block<K2, CB>(xr, tiles, stride_k, pr0, pr1, stage, lane, L, h, acc);
    TF_MARK(2);
    // D[row 4 kq + i][column c] of column tile j -> red[wave][row][16 j + c]
    __syncthreads();
    TF_MARK(3);
#pragma unroll
    for (int j = 0; j < 8; ++j)
#pragma unroll
      for (int i = 0; i < 4; ++i) red[(wave * 16 + 4 * kq + i) * 128 + 16 * j + c] = acc[j][i];
    __syncthreads();
    // a wave a row: the waves' sums in wave order, two columns a lane
    for (int r = wave; r < R; r += WK) {
      float2 s = *reinterpret_cast<const float2*>(red + r * 128 + 2 * lane);
      for (int w = 1; w < WK; ++w) {
        const float2 q = *reinterpret_cast<const float2*>(red + (w * 16 + r) * 128 + 2 * lane);
        s.x += q.x;
        s.y += q.y;
      }
      const size_t at = (size_t)(m0 + r) * N + col0 + 2 * lane;
      if (arrivals == 1) finish_row(s.x, s.y, lane, svh, bias, col0 + 2 * lane, y, y_dtype, at);
      else {
        // partial sums cross to another XCD's workgroup: agent-scope stores and loads are coherent by themselves
        // (a cache-wide write-back or invalidate, which __threadfence would issue, costs far more than the sums)
        float* zp = Z + (size_t)split * M * N + at;
        __hip_atomic_store(zp, s.x, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(zp + 1, s.y, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
    if (arrivals > 1) {
      __builtin_amdgcn_s_waitcnt(0);        // this wave's stores are acknowledged ...
      __syncthreads();                      // ... every wave's are ...
      TF_MARK(4);
      if (threadIdx.x == 0)                 // ... then the block counts itself in
        last = __hip_atomic_fetch_add(counters + (size_t)(pass * NB + nb) * TF_EXL3_COUNTER_STRIDE, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == arrivals - 1;
      __syncthreads();
      if (last) {
        // a row's sum over the K splits of the layer whose partial sums start at Zl: eight splits' loads go out
        // together (one trip to memory, not eight), then the sums in split order
        auto split_sums = [&](const float* Zl, size_t at, float& sx, float& sy) {
          sx = sy = 0.f;
          for (int q0 = 0; q0 < SK; q0 += 8) {
            float vx[8], vy[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) {
              const float* zq = Zl + (size_t)(q0 + j < SK ? q0 + j : SK - 1) * M * N + at;
              vx[j] = __hip_atomic_load(zq, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
              vy[j] = __hip_atomic_load(zq + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
#pragma unroll
            for (int j = 0; j < 8; ++j)
              if (q0 + j < SK) {
                sx = q0 + j ? sx + vx[j] : vx[j];
                sy = q0 + j ? sy + vy[j] : vy[j];
              }
          }
        };
        // the columns' scales are requested once, ahead of the rows' sums
        const int col = col0 + 2 * lane;
        const OutScale own(mlp ? svh0 : svh, mlp ? bias0 : bias, col);
        const OutScale other(svh0 + (mlp ? N : 0), mlp && bias0 ? bias0 + N : nullptr, col);       // up's, for an MLP
        float na = 0.f, nb2 = 0.f;
        if (mlp) load2(suh_next, TF_F16, col, na, nb2);
        for (int r = wave; r < R; r += WK) {
          const size_t at = (size_t)(m0 + r) * N + col;
          if (!mlp) {
            float sx, sy;
            split_sums(Z, at, sx, sy);
            finish_row(sx, sy, lane, own, y, y_dtype, at);
            continue;
          }
          float g0, g1, u0, u1;
          split_sums(Z0, at, g0, g1);
          split_sums(Z0 + (size_t)SK * M * N, at, u0, u1);
          finish_values(g0, g1, lane, own);
          finish_values(u0, u1, lane, other);
          if (y0) {
            store2(y0, y_dtype, at, g0, g1);
            store2(y0, y_dtype, (size_t)M * N + at, u0, u1);
          }
          swiglu_rot(g0, g1, u0, u1, y_dtype, lane, na, nb2, xh_next, at);
        }
        if (threadIdx.x == 0) counters[(size_t)(pass * NB + nb) * TF_EXL3_COUNTER_STRIDE] = 0;     // every block of the column has arrived
      }
    }
  }
  TF_MARK(5);
}

// W_q [K, N] fp16: a wave a tile
template <int K2, int CB>
__global__ void __launch_bounds__(64)
    unpack_kernel(const uint32_t* __restrict__ T, uint16_t* __restrict__ W, int N, int64_t stride_k, int64_t stride_nb) {
  const int kt = blockIdx.y, nt = blockIdx.x, lane = threadIdx.x, L = lane & 31, h = lane >> 5;
  const uint32_t* tile = T + (size_t)kt * stride_k + (size_t)(nt >> 3) * stride_nb + (nt & 7) * tile_words<K2>();
  uint16_t v[4];
  values4<K2, CB>(tile, L, h, v);
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int row = 2 * (L & 3) + (j & 1) + 8 * (j >> 1), col = (L >> 2) + 8 * h;
    W[(size_t)(kt * 16 + row) * N + nt * 16 + col] = v[j];
  }
}

// W_q as [K / 8][N][8] fp16, the order an MFMA B operand is read in: the 8 consecutive inputs a lane holds are 16
// bytes, and the 16 columns of a tile lie side by side, so a wave's operand load is four runs of 256 bytes.  A lane's
// four values are two pairs of consecutive inputs of one column: two 4-byte stores, a wave's a run of 256 bytes each.
// A workgroup takes four k-tiles of a 128-column block, a wave the eight tiles of one of them.
template <int K2, int CB>
__global__ void __launch_bounds__(256)
    unpack_k8_kernel(const uint32_t* __restrict__ T, uint16_t* __restrict__ W8, int N, int64_t stride_k,
                     int64_t stride_nb) {
  const int kt = 4 * blockIdx.y + (threadIdx.x >> 6), nb = blockIdx.x, lane = threadIdx.x & 63, L = lane & 31, h = lane >> 5;
  const uint32_t* tiles = T + (size_t)kt * stride_k + (size_t)nb * stride_nb;
  const int col = (L >> 2) + 8 * h;                      // values j = 0, 1: inputs 2 (L & 3), + 1; j = 2, 3: those + 8
  uint32_t* dst = reinterpret_cast<uint32_t*>(W8) + ((size_t)(2 * kt) * N + nb * 128 + col) * 4 + (L & 3);
#pragma unroll
  for (int t = 0; t < 8; ++t) {
    uint16_t v[4];
    values4<K2, CB>(tiles + t * tile_words<K2>(), L, h, v);
    dst[t * 64] = (uint32_t)v[0] | ((uint32_t)v[1] << 16);
    dst[(size_t)N * 4 + t * 64] = (uint32_t)v[2] | ((uint32_t)v[3] << 16);
  }
}

// ---- prompt matmul: y = ((xh @ W_q) H / sqrt(128)) * svh + bias on decoded weights (exl3/prefill.py:15-95) -----------
//
// xh fp16 [M, K] (rot_in's output), W8 fp16 [K / 8][N][8] (unpack_k8's).  A workgroup of WAVES waves takes 128 rows x
// 64 WAVES columns; a wave owns 64 columns = four B operands and all eight 16-row tiles, so one B operand feeds eight MFMAs
// and one LDS read of xh four: per 32 inputs a wave issues 32 MFMAs against 8 LDS reads and 4 global loads.  B
// operands come straight from W8 into registers (16 bytes a lane, 16 neighbouring lanes one 256-byte run: the cache
// sees 8 full lines a load, not 64 lanes' separate pieces), requested two steps of 64 inputs ahead; xh goes a step
// ahead through registers into LDS (two stages, 144-byte rows), one barrier a step.
// The epilogue is linear_kernel's: a row tile's sums through LDS, a wave a (row, 128-column block): FWHT, scale, bias.
// A row's arithmetic does not depend on the other rows, on M or on the tile it falls in.
//
// Workgroups reach the XCDs round-robin (blockIdx % 8) and each XCD has its own L2: the workgroups an XCD runs
// together (2^g_log2 consecutive ones) take an RG x CG block of tiles, so what they stream in step from beyond L2 is
// RG tiles of xh and CG of W8, not one of each a workgroup.
constexpr int GEMM_KSTEP = 64, GEMM_AROW = 2 * GEMM_KSTEP + 16, GEMM_STAGE = 128 * GEMM_AROW;     // bytes
constexpr int GEMM_LDS = 2 * GEMM_STAGE;         // two stages of xh; the epilogue's 16 x 516 floats fit too
static_assert(16 * 516 * 4 <= GEMM_LDS, "the epilogue's tile must fit the staging buffers");

template <int WAVES>
__global__ void __launch_bounds__(64 * WAVES, 8 / WAVES)
    gemm_kernel(const uint16_t* __restrict__ xh, const uint16_t* __restrict__ W8, const uint16_t* __restrict__ svh,
                const uint16_t* __restrict__ bias, void* __restrict__ y, int y_dtype, int64_t y_stride, int M, int K,
                int N, int rts, int cts, int rg_log2, int g_log2) {
  constexpr int THREADS = 64 * WAVES, COLS = 64 * WAVES, RED = COLS + 4;     // RED: floats a row of the epilogue's tile
  extern __shared__ __align__(16) unsigned char smem[];
  const int RG = 1 << rg_log2, CG = 1 << (g_log2 - rg_log2);
  const int xcd = blockIdx.x & 7, local = blockIdx.x >> 3;
  const int super = (local >> g_log2) * 8 + xcd, place = local & ((1 << g_log2) - 1);
  const int rgs = (rts + RG - 1) >> rg_log2;
  const int sc = super / rgs, sr = super - sc * rgs;
  const int rt = sr * RG + (place & (RG - 1)), ct = sc * CG + (place >> rg_log2);
  if (rt >= rts || ct >= cts) return;
  const int m0 = rt * 128, col0 = ct * COLS;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, c = lane & 15, kq = lane >> 4;
  const bool wok = col0 + 64 * wave < N;                   // N is a multiple of 128: a pair of waves falls out together
  const int steps = K / GEMM_KSTEP, last = steps - 1;

  // B: W8 from the workgroup's first column on as one buffer; the lane's octet and column as the vector offset, the
  // step's and chunk's octet as the scalar offset
  const int ncols = min(COLS, N - col0);
  const uint32_t octet = (uint32_t)N * 16u;                // bytes from one octet of inputs to the next
  const __amdgpu_buffer_rsrc_t wsrc = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<uint16_t*>(W8 + (size_t)col0 * 8), 0, (uint32_t)(K / 8 - 1) * octet + (uint32_t)ncols * 16u, 0x00020000);
  uint32_t boff[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) boff[j] = (uint32_t)kq * octet + (uint32_t)((wok ? 64 * wave : 0) + 16 * j + c) * 16u;
  typedef __attribute__((ext_vector_type(4))) uint32_t u32x4_t;
  u32x4_t b[2][4][2];
  auto load_b = [&](int step, int i, u32x4_t (&dst)[4][2]) {
#pragma unroll
    for (int j = 0; j < 4; ++j)
      dst[j][i] = __builtin_amdgcn_raw_buffer_load_b128(wsrc, boff[j], (step * 8 + 4 * i) * octet, 0);
  };
  // A: the workgroup's rows of xh as one buffer; this thread's 16-byte pieces of a step: piece q = (row q / 8,
  // 8 inputs q % 8); rows past M read the last row and are dropped at the end
  constexpr int PPT = 1024 / THREADS;
  const int nrows = min(128, M - m0);
  const __amdgpu_buffer_rsrc_t asrc = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<uint16_t*>(xh + (size_t)m0 * K), 0, (uint32_t)nrows * (uint32_t)K * 2u, 0x00020000);
  uint32_t aoff[PPT];
#pragma unroll
  for (int j = 0; j < PPT; ++j) {
    const int q = tid + THREADS * j;
    aoff[j] = ((uint32_t)min(q >> 3, nrows - 1) * (uint32_t)K + (q & 7) * 8) * 2u;
  }
  u32x4_t ar[PPT];
  auto load_a = [&](int step) {
#pragma unroll
    for (int j = 0; j < PPT; ++j) ar[j] = __builtin_amdgcn_raw_buffer_load_b128(asrc, aoff[j], step * (GEMM_KSTEP * 2), 0);
  };
  auto store_a = [&](int buf) {
#pragma unroll
    for (int j = 0; j < PPT; ++j) {
      const int q = tid + THREADS * j;
      *reinterpret_cast<u32x4_t*>(smem + buf * GEMM_STAGE + (q >> 3) * GEMM_AROW + (q & 7) * 16) = ar[j];
    }
  };

  f32x4_t acc[4][8];
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int r = 0; r < 8; ++r) acc[j][r] = (f32x4_t){0.f, 0.f, 0.f, 0.f};

  load_b(0, 0, b[0]);
  load_b(0, 1, b[0]);
  load_a(0);
  load_b(min(1, last), 0, b[1]);
  load_b(min(1, last), 1, b[1]);
  store_a(0);
  __syncthreads();
  // K is a multiple of 128, so the steps come in pairs: the loop body is one block with nothing conditional in it
  for (int step0 = 0; step0 < steps; step0 += 2) {
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int step = step0 + u;
      load_a(min(step + 1, last));
      __builtin_amdgcn_sched_barrier(0);                // the request leaves now, not when its registers are needed
      const unsigned char* abuf = smem + u * GEMM_STAGE + c * GEMM_AROW + kq * 16;
      // operand t of the step is (chunk t / 8, row tile t % 8), requested two row tiles before its MFMAs
      auto read_a = [&](int t) {
        return *reinterpret_cast<const f16x8_t*>(abuf + 16 * (t & 7) * GEMM_AROW + (t >> 3) * 64);
      };
      f16x8_t a = read_a(0), a1 = read_a(1);
#pragma unroll
      for (int i = 0; i < 2; ++i) {
#pragma unroll
        for (int r = 0; r < 8; ++r) {
          const int t = 8 * i + r;
          f16x8_t a2 = a1;
          if (t + 2 < 16) a2 = read_a(t + 2);
#pragma unroll
          for (int j = 0; j < 4; ++j)
            acc[j][r] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, __builtin_bit_cast(f16x8_t, b[u][j][i]), acc[j][r], 0, 0, 0);
          a = a1;
          a1 = a2;
          // keep the order written here: one LDS read two row tiles ahead of the four MFMAs it feeds
          if (t == 0) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
          if (t + 2 < 16) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
        load_b(min(step + 2, last), i, b[u]);           // this chunk's registers are free again
        __builtin_amdgcn_sched_barrier(0);
      }
      store_a(1 - u);
      __syncthreads();
    }
  }
  // D[row 4 kq + e][column c] of tile (j, r) -> LDS [16 rows][RED] a row tile at a time, then a wave a (row, block)
  float* red = reinterpret_cast<float*>(smem);
#pragma unroll
  for (int r = 0; r < 8; ++r) {
    if (r) __syncthreads();
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int e = 0; e < 4; ++e) red[(4 * kq + e) * RED + 64 * wave + 16 * j + c] = acc[j][r][e];
    __syncthreads();
    for (int unit = wave; unit < 8 * WAVES; unit += WAVES) {
      const int row = unit / (WAVES / 2), blk = unit % (WAVES / 2);
      const int grow = m0 + 16 * r + row, col = col0 + 128 * blk + 2 * lane;
      if (grow < M && col0 + 128 * blk < N) {
        const float2 v = *reinterpret_cast<const float2*>(red + row * RED + 128 * blk + 2 * lane);
        finish_row(v.x, v.y, lane, svh, bias, col, y, y_dtype, (size_t)grow * y_stride + col);
      }
    }
  }
}


}  // namespace
}  // namespace tf

using namespace tf;

static int rot_in_launch(const char* who, const void* x, int x_dtype, const uint16_t* suh, uint16_t* xh, int layers,
                         int m, int k, tf_stream_t stream) {
  clear_error();
  TF_REQUIRE(x && suh && xh, "%s: null pointer argument", who);
  TF_REQUIRE(x_dtype == TF_F16 || x_dtype == TF_BF16 || x_dtype == TF_F32, "x: expected fp16, bf16 or fp32");
  TF_REQUIRE(m >= 1 && k >= 128 && k % 128 == 0, "x and xh must be [M, K], K a multiple of 128, suh [K]");
  TF_REQUIRE(layers >= 1 && layers <= 64, "%s: 1 to 64 layers a stack", who);
  TF_REQUIRE(aligned16(x) && aligned16(xh), "x: must be 16-byte aligned");
  rot_in_kernel<<<dim3((k / 128 + 3) / 4, m < 1024 ? m : 1024, layers), 256, 0, as_stream(stream)>>>(x, x_dtype, suh, xh, m, k);
  TF_LAUNCH_OK(who);
  return 0;
}

extern "C" int tf_exl3_rot_in(const void* x, int x_dtype, const uint16_t* suh, uint16_t* xh, int m, int k,
                              tf_stream_t stream) {
  return rot_in_launch("tf_exl3_rot_in", x, x_dtype, suh, xh, 1, m, k, stream);
}

extern "C" int tf_exl3_rot_in_stacked(const void* x, int x_dtype, const uint16_t* suh, uint16_t* xh, int layers, int m,
                                      int k, tf_stream_t stream) {
  return rot_in_launch("tf_exl3_rot_in_stacked", x, x_dtype, suh, xh, layers, m, k, stream);
}

TF_TIMELINE_EXPORT(exl3)

static int linear_launch(const char* who, const uint16_t* xh, const uint32_t* T, int64_t stride_k, int64_t stride_nb,
                         int64_t stride_layer, const uint16_t* svh, const uint16_t* bias, void* y, int y_dtype, float* Z,
                         int32_t* counters, int layers, int m, int k, int n, int k2, int cb, int sk, int wk,
                         tf_stream_t stream, const uint16_t* suh_next = nullptr, uint16_t* xh_next = nullptr) {
  clear_error();
  TF_REQUIRE(xh && T && svh && (y || xh_next), "%s: null pointer argument", who);
  TF_REQUIRE(!xh_next || (layers == 2 && suh_next && Z && counters && aligned16(xh_next)),
             "%s: the SwiGLU needs two layers (gate, up), the next layer's suh, Z and counters", who);
  TF_REQUIRE(y_dtype == TF_F16 || y_dtype == TF_BF16 || y_dtype == TF_F32, "y: expected fp16, bf16 or fp32");
  TF_REQUIRE(m >= 1 && m <= 128, "xh and y must have the same 1 to 128 rows");
  TF_REQUIRE(k >= 128 && n >= 128 && k % 128 == 0 && n % 128 == 0, "K and N must be multiples of 128");
  TF_REQUIRE(aligned16(T) && aligned16(xh) && aligned16(y), "T must be 16-byte aligned");          // (a null y is aligned)
  TF_REQUIRE(layers >= 1 && layers <= 64 && (layers == 1 || (stride_layer > 0 && stride_layer % 4 == 0)),
             "%s: 1 to 64 layers, a whole number of 16-byte pieces apart", who);
  TF_REQUIRE(layers == 1 || ((int64_t)m * k % 8 == 0 && (int64_t)m * n % 8 == 0), "%s: layers' xh and y must stay 16-byte aligned", who);
  TF_REQUIRE(wk == 2 || wk == 4 || wk == 8, "WK must be 2, 4 or 8");
  TF_REQUIRE(sk >= 1 && sk <= 64 && (int64_t)sk * wk <= k / 32, "K / 32 = %d tile pairs do not split over %d x %d waves",
             k / 32, sk, wk);
  TF_REQUIRE(sk == 1 || (Z && counters), "Z and counters are needed with more than one split");
  const dim3 grid((unsigned)(n / 128), (unsigned)sk, (unsigned)layers);
  hipStream_t s = as_stream(stream);
  const size_t smem = (size_t)wk * 16 * 128 * sizeof(float);
#define TF_LAUNCH(K2_, CB_)                                                                                             \
  if (k2 == K2_ && cb == CB_) {                                                                                         \
    if (wk == 2) linear_kernel<K2_, CB_, 2><<<grid, 128, smem, s>>>(xh, T, stride_k, stride_nb, stride_layer, svh, bias, y, y_dtype, Z, counters, m, k, n, sk, suh_next, xh_next); \
    else if (wk == 4) linear_kernel<K2_, CB_, 4><<<grid, 256, smem, s>>>(xh, T, stride_k, stride_nb, stride_layer, svh, bias, y, y_dtype, Z, counters, m, k, n, sk, suh_next, xh_next); \
    else linear_kernel<K2_, CB_, 8><<<grid, 512, smem, s>>>(xh, T, stride_k, stride_nb, stride_layer, svh, bias, y, y_dtype, Z, counters, m, k, n, sk, suh_next, xh_next); \
    TF_LAUNCH_OK(who);                                                                                                  \
    return 0;                                                                                                           \
  }
  TF_EXL3_ALL(TF_LAUNCH)
#undef TF_LAUNCH
  set_error("unsupported EXL3 width/codebook: K2=%d codebook=%d", k2, cb);
  return 1;
}

extern "C" int tf_exl3_linear(const uint16_t* xh, const uint32_t* T, int64_t stride_k, int64_t stride_nb,
                              const uint16_t* svh, const uint16_t* bias, void* y, int y_dtype, float* Z,
                              int32_t* counters, int m, int k, int n, int k2, int cb, int sk, int wk,
                              tf_stream_t stream) {
  return linear_launch("tf_exl3_linear", xh, T, stride_k, stride_nb, 0, svh, bias, y, y_dtype, Z, counters, 1, m, k, n,
                       k2, cb, sk, wk, stream);
}

extern "C" int tf_exl3_linear_stacked(const uint16_t* xh, const uint32_t* T, int64_t stride_k, int64_t stride_nb,
                                      int64_t stride_layer, const uint16_t* svh, const uint16_t* bias, void* y,
                                      int y_dtype, float* Z, int32_t* counters, int layers, int m, int k, int n, int k2,
                                      int cb, int sk, int wk, tf_stream_t stream) {
  return linear_launch("tf_exl3_linear_stacked", xh, T, stride_k, stride_nb, stride_layer, svh, bias, y, y_dtype, Z,
                       counters, layers, m, k, n, k2, cb, sk, wk, stream);
}

extern "C" int tf_exl3_gate_up(const uint16_t* xh, const uint32_t* T, int64_t stride_k, int64_t stride_nb,
                               int64_t stride_layer, const uint16_t* svh, const uint16_t* bias, void* y, int y_dtype,
                               float* Z, int32_t* counters, const uint16_t* suh_next, uint16_t* xh_next, int m, int k,
                               int n, int k2, int cb, int sk, int wk, tf_stream_t stream) {
  clear_error();
  TF_REQUIRE(suh_next && xh_next, "tf_exl3_gate_up: null pointer argument");
  return linear_launch("tf_exl3_gate_up", xh, T, stride_k, stride_nb, stride_layer, svh, bias, y, y_dtype, Z, counters, 2, m,
                       k, n, k2, cb, sk, wk, stream, suh_next, xh_next);
}

extern "C" int tf_exl3_swiglu_rot_in(const void* y, int y_dtype, const uint16_t* suh, uint16_t* xh, int m, int n,
                                     tf_stream_t stream) {
  clear_error();
  TF_REQUIRE(y && suh && xh, "tf_exl3_swiglu_rot_in: null pointer argument");
  TF_REQUIRE(y_dtype == TF_F16 || y_dtype == TF_BF16 || y_dtype == TF_F32, "y: expected fp16, bf16 or fp32");
  TF_REQUIRE(m >= 1 && n >= 128 && n % 128 == 0, "y must be [2, M, N], N a multiple of 128, suh [N]");
  TF_REQUIRE(aligned16(y) && aligned16(xh) && (int64_t)m * n % 8 == 0, "y and xh must be 16-byte aligned");
  swiglu_rot_in_kernel<<<dim3((n / 128 + 3) / 4, m < 1024 ? m : 1024), 256, 0, as_stream(stream)>>>(y, y_dtype, suh, xh, m, n);
  TF_LAUNCH_OK("tf_exl3_swiglu_rot_in");
  return 0;
}

extern "C" int tf_exl3_unpack(const uint32_t* T, uint16_t* W, int k, int n, int64_t stride_k, int64_t stride_nb, int k2,
                              int cb, tf_stream_t stream) {
  clear_error();
  TF_REQUIRE(T && W, "unpack: null pointer argument");
  TF_REQUIRE(k >= 128 && n >= 128 && k % 128 == 0 && n % 128 == 0, "W must be [K, N], multiples of 128");
  TF_REQUIRE(k / 16 <= 65535, "unpack: K too large for one launch");
  const dim3 grid((unsigned)(n / 16), (unsigned)(k / 16));
  hipStream_t s = as_stream(stream);
#define TF_LAUNCH(K2_, CB_)                                                          \
  if (k2 == K2_ && cb == CB_) {                                                      \
    unpack_kernel<K2_, CB_><<<grid, 64, 0, s>>>(T, W, n, stride_k, stride_nb);       \
    TF_LAUNCH_OK("tf_exl3_unpack");                                                  \
    return 0;                                                                        \
  }
  TF_EXL3_EVERY(TF_LAUNCH)
#undef TF_LAUNCH
  set_error("unsupported EXL3 width/codebook: K2=%d codebook=%d", k2, cb);
  return 1;
}

extern "C" int tf_exl3_unpack_k8(const uint32_t* T, uint16_t* W8, int k, int n, int64_t stride_k, int64_t stride_nb,
                                 int k2, int cb, tf_stream_t stream) {
  clear_error();
  TF_REQUIRE(T && W8 && aligned16(W8), "unpack_k8: null or unaligned pointer argument");
  TF_REQUIRE(k >= 128 && n >= 128 && k % 128 == 0 && n % 128 == 0, "W must be [K, N], multiples of 128");
  TF_REQUIRE(k / 64 <= 65535, "unpack_k8: K too large for one launch");
  const dim3 grid((unsigned)(n / 128), (unsigned)(k / 64));
  hipStream_t s = as_stream(stream);
#define TF_LAUNCH(K2_, CB_)                                                            \
  if (k2 == K2_ && cb == CB_) {                                                        \
    unpack_k8_kernel<K2_, CB_><<<grid, 256, 0, s>>>(T, W8, n, stride_k, stride_nb);    \
    TF_LAUNCH_OK("tf_exl3_unpack_k8");                                                 \
    return 0;                                                                          \
  }
  TF_EXL3_ALL(TF_LAUNCH)
#undef TF_LAUNCH
  set_error("unsupported EXL3 width/codebook: K2=%d codebook=%d", k2, cb);
  return 1;
}

extern "C" int tf_exl3_gemm(const uint16_t* xh, const uint16_t* w8, const uint16_t* svh, const uint16_t* bias, void* y,
                            int y_dtype, int64_t y_stride, int m, int k, int n, tf_stream_t stream) {
  clear_error();
  TF_REQUIRE(xh && w8 && svh && y, "gemm: null pointer argument");
  TF_REQUIRE(m >= 1 && k >= 128 && n >= 128 && k % 128 == 0 && n % 128 == 0, "xh [M, K], W8 [K / 8, N, 8]: multiples of 128");
  TF_REQUIRE((int64_t)k * n < (1LL << 31), "gemm: K * N must stay below 2^31 (buffer offsets are 32-bit)");
  TF_REQUIRE(y_dtype == TF_F16 || y_dtype == TF_BF16 || y_dtype == TF_F32, "y: expected fp16, bf16 or fp32");
  TF_REQUIRE(y_stride >= n && y_stride % 2 == 0, "y rows hold at least N values, an even stride apart");
  TF_REQUIRE(aligned16(xh) && aligned16(w8) && ((uintptr_t)y & 7) == 0, "xh, W8 16-byte and y 8-byte aligned");
  // 128 x 256 tiles, four waves, two workgroups a CU: one workgroup's first loads and its epilogue run under the
  // other's MFMAs, and the last, part-filled round of tiles is spread thinner
  constexpr int WAVES = 4, COLS = 64 * WAVES;
  const int64_t rts = ((int64_t)m + 127) / 128, cts = (n + COLS - 1) / COLS;
  TF_REQUIRE(rts <= 0x3FFFFF, "gemm: too many rows for one launch");
  // an XCD's 2^g_log2 consecutive workgroups: 2^rg_log2 row tiles x the rest column tiles; smaller groups when the
  // whole grid would not give every XCD two of them
  int g_log2 = WAVES == 4 ? 6 : 5, rg_log2 = 0;
  int64_t supers = 0;
  for (;; --g_log2) {
    rg_log2 = 0;
    while (rg_log2 < 3 && rg_log2 < g_log2 && (1 << rg_log2) < rts) ++rg_log2;
    const int64_t cg = 1 << (g_log2 - rg_log2);
    supers = ((rts + (1 << rg_log2) - 1) >> rg_log2) * ((cts + cg - 1) / cg);
    if (supers >= 16 || g_log2 == 3) break;
  }
  const int64_t grid = (supers + 7) / 8 * (8 << g_log2);
  TF_REQUIRE(grid <= 0x7FFFFFFF, "gemm: %lld workgroups exceed the grid limit", (long long)grid);
  gemm_kernel<WAVES><<<dim3((unsigned)grid), 64 * WAVES, GEMM_LDS, as_stream(stream)>>>(
      xh, w8, svh, bias, y, y_dtype, y_stride, m, k, n, (int)rts, (int)cts, rg_log2, g_log2);
  TF_LAUNCH_OK("tf_exl3_gemm");
  return 0;
}
