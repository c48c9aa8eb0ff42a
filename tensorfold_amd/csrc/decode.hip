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
#include <mutex>

#include "gemv.h"
#include "routing.h"

namespace tf {
namespace {

// A workgroup takes (item, pair of 32-column blocks, RBMAX of the item's rows): one pass over its weights, as with
// item descriptors.  (Taking all of an item's up to 16 rows made it stream the same weights up to eight times, and
// a compute unit's workgroups together overflow the L2 between passes.)  blockIdx.y picks the rows; see expert_unit.
template <int GS, int NM, int EPI, int WAVES>
__global__ void __launch_bounds__(WAVES * 64)
    expert_kernel(const uint16_t* __restrict__ X, int64_t x_stride, int slots, const uint32_t* __restrict__ W, int KG,
                  int NB, const int* __restrict__ items, const int* __restrict__ counts,
                  const int* __restrict__ members, void* __restrict__ out, int N, float limit) {
  extern __shared__ float lds[];
  const int NB2 = (NB + 1) >> 1;
  const int it = blockIdx.x / NB2, cb2 = blockIdx.x - it * NB2;
  if (it >= counts[0]) return;
  const int e = items[3 * it], first = items[3 * it + 1], total = items[3 * it + 2];
  NoHook none;
  // rows RBMAX y .. of every 16 (a decode item holds at most 16, so this runs once)
  for (int skip = RBMAX * blockIdx.y; skip < total; skip += RBMAX * gridDim.y) {
    if (skip != RBMAX * (int)blockIdx.y) __syncthreads();
    expert_unit<GS, NM, EPI, WAVES, 0>(X, x_stride, slots, W, KG, NB, e, min(RBMAX, total - skip),
                                       members + first + skip, cb2, out, N, limit, lds, none);
  }
}

// The same unit taken from an item descriptor as tf_moe_route_decode and tf_moe_route_up write them: one read
// instead of the items -> members chain, and items of at most DTILE pairs.
template <int GS, int NM, int EPI, int WAVES>
__global__ void __launch_bounds__(WAVES * 64)
    expert_desc_kernel(const uint16_t* __restrict__ X, int64_t x_stride, int slots, const uint32_t* __restrict__ W,
                       int KG, int NB, const int* __restrict__ desc, const int* __restrict__ counts,
                       void* __restrict__ out, int N, float limit) {
  extern __shared__ float lds[];
  __shared__ int pairs[16];
  const int NB2 = (NB + 1) >> 1;
  const int it = blockIdx.x / NB2, cb2 = blockIdx.x - it * NB2;
  // the descriptor's words are requested with the count, not after it (a row past the count exists and is ignored)
  const int* d = desc + (size_t)(1 + it) * DESC;
  const int n_items = desc[0], e = d[0], cnt = d[1], p0 = d[4], p1 = d[5];
  if (it >= n_items) return;
  if (threadIdx.x < DTILE) pairs[threadIdx.x] = threadIdx.x ? p1 : p0;
  __syncthreads();
  NoHook none;
  expert_unit<GS, NM, EPI, WAVES, 0>(X, x_stride, slots, W, KG, NB, e, cnt, pairs, cb2, out, N, limit, lds, none);
}

// ---- dense lane matmul ---------------------------------------------------------------------------------------------

constexpr int QRB = 8;          // rows a pass of the dense split kernels (the one-launch form keeps pairs)

struct NoFlush {
  template <class A>
  __device__ __forceinline__ void operator()(int, A&) const {}
};

// One pass of a row tile: RB rows r0 .. r0 + RB - 1 against the workgroup's 64 columns and K slice.
template <int GS, int WAVES, int RB, bool COH, class WQ, class SB>
__device__ __forceinline__ void qmm_pass(const uint16_t* __restrict__ X, int64_t ldx, const float* __restrict__ XS,
                                         const WQ& wq, const SB& sb, int r0, int tile, int slice, int gs0, int per,
                                         int g0, int g1, void* __restrict__ out, float* __restrict__ part_out, int M,
                                         int N, int KG, int SK, int f32, float* xs, float* part,
                                         Stage<GS, 1, QRB> (&st)[DEPTH], bool loaded, int valid) {
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const uint32_t* xl[RB];
  const_u32_ptr xsr[RB];
#pragma unroll
  for (int r = 0; r < RB; ++r) {
    const int row = r0 + (r < valid ? r : valid - 1);          // a pass past the last row walks that row again, unstored
    xl[r] = reinterpret_cast<const uint32_t*>(X + (size_t)row * ldx) + (lane & 15);
    xsr[r] = as_const(XS + (size_t)row * KG);
  }
  __syncthreads();                                  // the previous pass is done with part
  float acc[1][RB];
#pragma unroll
  for (int r = 0; r < RB; ++r) acc[0][r] = 0.f;
  NoFlush none;
  auto xsum = [&](int r, int g) { return __uint_as_float(xsr[r][g]); };
  gemv_stream<GS, 1, RB, 0>(acc, st, loaded, wq, sb, xl, xsum, g0, g1, none);
#pragma unroll
  for (int r = 0; r < RB; ++r) part[(wave * RB + r) * 64 + lane] = acc[0][r];
  __syncthreads();
  for (int o = tid; o < valid * 64; o += WAVES * 64) {
    const int r = o >> 6, l = o & 63, cc = tile * 64 + l;
    if (cc >= N) continue;
    float s = part[r * 64 + l];
    for (int w = 1; w < WAVES; ++w) s += part[(w * RB + r) * 64 + l];
    const size_t at = (size_t)(r0 + r) * N + cc;
    if (SK > 1) {
      // COH: another workgroup adds the slices up in this launch: the store goes through to where it can read it
      if (COH) __hip_atomic_store(part_out + (size_t)slice * M * N + at, s, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      else part_out[(size_t)slice * M * N + at] = s;
    } else if (f32) reinterpret_cast<float*>(out)[at] = s;
    else reinterpret_cast<uint16_t*>(out)[at] = (uint16_t)f32_bf16_bits(s);
  }
}

// grid (column tiles of 64 x row tiles of BM, 1, SK).  Slice z takes groups [z * per, (z + 1) * per), its waves
// split them again (added in wave order); SK > 1 leaves the slice's fp32 sums in part[z].  Rows go in passes of 8, 4,
// 2 or 1 (a row's arithmetic is the same in each: what a pass shares is the unpacked weights); 5 to 7 rows take the
// pass of 8 and 3 rows the pass of 4, rather than two passes over the weights.
template <int GS, int WAVES, bool COH = false>
__device__ __forceinline__ void qmm_block(const uint16_t* __restrict__ X, int64_t ldx, const float* __restrict__ XS,
                                          const uint32_t* __restrict__ W, const uint16_t* __restrict__ S,
                                          const uint16_t* __restrict__ B, int64_t sb_stride, void* __restrict__ out,
                                          float* __restrict__ part_out, int M, int N, int KG, int SK, int BM, int f32,
                                          int block, int slice, float* lds) {
  const int tiles = (N + 63) >> 6;
  const int tile = block % tiles, rt = block / tiles;
  const int per = KG / SK, gs0 = slice * per;
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  constexpr int CH = GS / 32;
  const uint32_t* wbase = W + ((size_t)tile * KG) * (size_t)(CH * 256) + lane * 4;
  const int col = tile * 64 + lane;
  auto wq = [&](int g, int m, int i) { return ldg16(wbase + ((size_t)g * CH + i) * 256); };
  auto sb = [&](int g, int m, uint32_t& s, uint32_t& b) {
    s = S[(size_t)g * sb_stride + col];
    b = B[(size_t)g * sb_stride + col];
  };
  const int g0 = gs0 + (int)((long long)wave * per / WAVES), g1 = gs0 + (int)((long long)(wave + 1) * per / WAVES);
  float* xs = nullptr;
  float* part = lds;
  const int m_end = min(M, (rt + 1) * BM);
  int r0 = rt * BM;
  Stage<GS, 1, QRB> st[DEPTH];
#pragma unroll
  for (int d = 0; d < DEPTH; ++d)
    if (g0 + d < g1) load_weights<GS, 1>(st[d], wq, sb, g0 + d);
  bool loaded = true;
#define TF_QMM_PASS(RB_)                                                                                             \
  {                                                                                                                  \
    const int valid = min(RB_, m_end - r0);                                                                          \
    qmm_pass<GS, WAVES, RB_, COH>(X, ldx, XS, wq, sb, r0, tile, slice, gs0, per, g0, g1, out, part_out, M, N, KG, SK, \
                                  f32, xs, part, st, loaded, valid);                                                 \
    loaded = g1 - g0 <= DEPTH;                                                                                       \
    r0 += valid;                                                                                                     \
  }
  while (m_end - r0 >= 5) TF_QMM_PASS(8)
  if (m_end - r0 >= 3) TF_QMM_PASS(4)
  if (m_end - r0 == 2) TF_QMM_PASS(2)
  if (m_end - r0 == 1) TF_QMM_PASS(1)
#undef TF_QMM_PASS
}

template <int GS, int WAVES>
__global__ void __launch_bounds__(WAVES * 64)
    qmm_kernel(const uint16_t* __restrict__ X, int64_t ldx, const float* __restrict__ XS,
               const uint32_t* __restrict__ W, const uint16_t* __restrict__ S, const uint16_t* __restrict__ B,
               int64_t sb_stride, void* __restrict__ out, float* __restrict__ part_out, int M, int N, int KG, int SK,
               int BM, int f32) {
  extern __shared__ float lds[];            // partials [WAVES][QRB][64]
  qmm_block<GS, WAVES>(X, ldx, XS, W, S, B, sb_stride, out, part_out, M, N, KG, SK, BM, f32, blockIdx.x, blockIdx.z, lds);
}

// The split matmul with its reduce in the same launch: a slice's workgroup leaves its sums in part[z] with stores
// that go through to memory, waits for them to be acknowledged and counts itself in at the (column tile, row tile)'s
// counter; the workgroup that finds the others there adds the slices in slice order (qmm_reduce_kernel's arithmetic)
// and puts the counter back to zero.  A thousand short workgroups fill the chip where the one-launch form above has
// one workgroup a column tile.
// What a slice's workgroup does once its sums are in part[z] (stored through to memory): wait for the stores'
// acknowledgement, count itself in at the tile's counter, and if every other slice is there already add them up.
template <int WAVES>
__device__ __forceinline__ void qmm_arrive_tail(int* __restrict__ counter, const float* __restrict__ part_out,
                                                void* __restrict__ out, int M, int N, int SK, int BM, int f32, int block,
                                                int* last) {
  __builtin_amdgcn_s_waitcnt(0);        // this wave's stores are acknowledged ...
  __syncthreads();                      // ... every wave's are ...
  if (threadIdx.x == 0)                 // ... then the workgroup counts itself in
    *last = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == SK - 1;
  __syncthreads();
  if (!*last) return;
  const int tiles = (N + 63) >> 6, tile = block % tiles, rt = block / tiles;
  const int r_first = rt * BM, rows = min(M, r_first + BM) - r_first;
  const long long total = (long long)M * N;
  for (int o = threadIdx.x; o < rows * 64; o += WAVES * 64) {
    const int cc = tile * 64 + (o & 63);
    if (cc >= N) continue;
    const size_t at = (size_t)(r_first + (o >> 6)) * N + cc;
    // eight slices' loads go out together, then the sums in slice order
    float acc = 0.f;
    for (int z0 = 0; z0 < SK; z0 += 8) {
      float v[8];
#pragma unroll
      for (int j = 0; j < 8; ++j)
        v[j] = __hip_atomic_load(part_out + (long long)(z0 + j < SK ? z0 + j : SK - 1) * total + at, __ATOMIC_RELAXED,
                                 __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
      for (int j = 0; j < 8; ++j)
        if (z0 + j < SK) acc = z0 + j ? acc + v[j] : v[j];
    }
    if (f32) reinterpret_cast<float*>(out)[at] = acc;
    else reinterpret_cast<uint16_t*>(out)[at] = (uint16_t)f32_bf16_bits(acc);
  }
  if (threadIdx.x == 0) *counter = 0;   // every slice of the tile has arrived: ready for the next call
}

template <int GS, int WAVES>
__global__ void __launch_bounds__(WAVES * 64)
    qmm_arrive_kernel(const uint16_t* __restrict__ X, int64_t ldx, const float* __restrict__ XS,
                      const uint32_t* __restrict__ W, const uint16_t* __restrict__ S, const uint16_t* __restrict__ B,
                      int64_t sb_stride, void* __restrict__ out, float* __restrict__ part_out, int* __restrict__ counters,
                      int M, int N, int KG, int SK, int BM, int f32) {
  extern __shared__ float lds[];
  __shared__ int last;
  qmm_block<GS, WAVES, true>(X, ldx, XS, W, S, B, sb_stride, out, part_out, M, N, KG, SK, BM, f32, blockIdx.x, blockIdx.z, lds);
  qmm_arrive_tail<WAVES>(counters + (size_t)blockIdx.x * TF_QMM_COUNTER_STRIDE, part_out, out, M, N, SK, BM, f32,
                         blockIdx.x, &last);
}

// The split matmul and its reduce in ONE launch, with no traffic between workgroups: a workgroup of FW waves takes a
// (column tile, row tile) with ALL of K.  The 4 * SK sub-slices (SK slices x the 4 waves qmm_kernel runs a slice on)
// keep their boundaries; wave w streams 4 * SK / FW consecutive ones, parking each sum in LDS, and the end adds a
// slice's four in wave order, then the slices in slice order: the arithmetic, and so the bits, of qmm_kernel followed
// by qmm_reduce_kernel.  The same waves are in flight as in the split launch; only the grouping differs.
template <int GS, int FW, int RB, class WQ, class SB>
__device__ __forceinline__ void qmm_fat_pass(const uint16_t* __restrict__ X, int64_t ldx, const float* __restrict__ XS,
                                             const WQ& wq, const SB& sb, int r0, int tile, int per, int SK, int gA,
                                             int gB, void* __restrict__ out, int N, int KG, int f32, float* part,
                                             Stage<GS, 1> (&st)[DEPTH], bool loaded) {
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int U = 4 * SK, SPW = U / FW;
  auto sub_begin = [&](int u) { return (u >> 2) * per + (int)((long long)(u & 3) * per / 4); };
  const uint32_t* xl[RB];
  const_u32_ptr xsr[RB];
#pragma unroll
  for (int r = 0; r < RB; ++r) {
    xl[r] = reinterpret_cast<const uint32_t*>(X + (size_t)(r0 + r) * ldx) + (lane & 15);
    xsr[r] = as_const(XS + (size_t)(r0 + r) * KG);
  }
  __syncthreads();                                  // the previous pass is done with part
  if (per < 4) {                                    // sub-slices with no group still take part in the sums: as zeros
    for (int q = 0; q < SPW; ++q)
#pragma unroll
      for (int r = 0; r < RB; ++r) part[((wave * SPW + q) * RB + r) * 64 + lane] = 0.f;
  }
  float acc[1][RB];
#pragma unroll
  for (int r = 0; r < RB; ++r) acc[0][r] = 0.f;
  int sub = wave * SPW;
  const int sub_last = (wave + 1) * SPW;
  while (sub < sub_last && sub_begin(sub + 1) == sub_begin(sub)) ++sub;
  int sub_end = sub < sub_last ? sub_begin(sub + 1) : -1;
  auto flush = [&](int g, float (&a)[1][RB]) {
    if (g + 1 != sub_end) return;
#pragma unroll
    for (int r = 0; r < RB; ++r) {
      part[(sub * RB + r) * 64 + lane] = a[0][r];
      a[0][r] = 0.f;
    }
    ++sub;
    while (sub < sub_last && sub_begin(sub + 1) == sub_begin(sub)) ++sub;
    sub_end = sub < sub_last ? sub_begin(sub + 1) : -1;
  };
  auto xsum = [&](int r, int g) { return __uint_as_float(xsr[r][g]); };
  gemv_stream<GS, 1, RB, 0>(acc, st, loaded, wq, sb, xl, xsum, gA, gB, flush);
  __syncthreads();
  for (int o = tid; o < RB * 64; o += FW * 64) {
    const int r = o >> 6, l = o & 63, cc = tile * 64 + l;
    if (cc >= N) continue;
    float total = 0.f;
    for (int z = 0; z < SK; ++z) {
      float t = part[((4 * z) * RB + r) * 64 + l];
      for (int j = 1; j < 4; ++j) t += part[((4 * z + j) * RB + r) * 64 + l];
      total = z ? total + t : t;
    }
    const size_t at = (size_t)(r0 + r) * N + cc;
    if (f32) reinterpret_cast<float*>(out)[at] = total;
    else reinterpret_cast<uint16_t*>(out)[at] = (uint16_t)f32_bf16_bits(total);
  }
}

template <int GS, int FW>
__device__ __forceinline__ void qmm_fat_block(const uint16_t* __restrict__ X, int64_t ldx, const float* __restrict__ XS,
                                              const uint32_t* __restrict__ W, const uint16_t* __restrict__ S,
                                              const uint16_t* __restrict__ B, int64_t sb_stride,
                                              void* __restrict__ out, int M, int N, int KG, int SK, int BM, int f32,
                                              int block, float* lds) {
  const int tiles = (N + 63) >> 6;
  const int tile = block % tiles, rt = block / tiles;
  const int per = KG / SK;
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  constexpr int CH = GS / 32;
  const uint32_t* wbase = W + ((size_t)tile * KG) * (size_t)(CH * 256) + lane * 4;
  const int col = tile * 64 + lane;
  auto wq = [&](int g, int m, int i) { return ldg16(wbase + ((size_t)g * CH + i) * 256); };
  auto sb = [&](int g, int m, uint32_t& s, uint32_t& b) {
    s = S[(size_t)g * sb_stride + col];
    b = B[(size_t)g * sb_stride + col];
  };
  auto sub_begin = [&](int u) { return (u >> 2) * per + (int)((long long)(u & 3) * per / 4); };
  const int SPW = 4 * SK / FW;
  const int gA = sub_begin(wave * SPW), gB = sub_begin((wave + 1) * SPW);
  const int m_end = min(M, (rt + 1) * BM);
  int r0 = rt * BM;
  Stage<GS, 1> st[DEPTH];
#pragma unroll
  for (int d = 0; d < DEPTH; ++d)
    if (gA + d < gB) load_weights<GS, 1>(st[d], wq, sb, gA + d);
  bool loaded = true;
  for (; r0 + 2 <= m_end; r0 += 2) {
    qmm_fat_pass<GS, FW, 2>(X, ldx, XS, wq, sb, r0, tile, per, SK, gA, gB, out, N, KG, f32, lds, st, loaded);
    loaded = gB - gA <= DEPTH;
  }
  if (r0 < m_end) qmm_fat_pass<GS, FW, 1>(X, ldx, XS, wq, sb, r0, tile, per, SK, gA, gB, out, N, KG, f32, lds, st, loaded);
}

template <int GS, int FW>
__global__ void __launch_bounds__(FW * 64)
    qmm_fat_kernel(const uint16_t* __restrict__ X, int64_t ldx, const float* __restrict__ XS,
                   const uint32_t* __restrict__ W, const uint16_t* __restrict__ S, const uint16_t* __restrict__ B,
                   int64_t sb_stride, void* __restrict__ out, int M, int N, int KG, int SK, int BM, int f32) {
  extern __shared__ float lds[];            // sub-slice sums [4 * SK][RBMAX][64]
  qmm_fat_block<GS, FW>(X, ldx, XS, W, S, B, sb_stride, out, M, N, KG, SK, BM, f32, blockIdx.x, lds);
}

// Up to four weights against one x in one launch (and one reduce launch): workgroups [first[w], first[w + 1]) take
// weight w's (column tile, row tile) pairs; grid.z is the largest slice count and a weight's surplus slices leave.
constexpr int GROUP_MAX = 4;
struct GroupArgs {
  const uint32_t* w[GROUP_MAX];
  const uint16_t* s[GROUP_MAX];
  const uint16_t* b[GROUP_MAX];
  void* out[GROUP_MAX];
  float* part[GROUP_MAX];
  int* counters[GROUP_MAX];      // arrival counters of a weight (the arriving form), else unused
  int64_t sb_stride[GROUP_MAX];
  int n[GROUP_MAX], sk[GROUP_MAX];
  int first[GROUP_MAX + 1];      // workgroups (matmul) or 256-element chunks (reduce) before weight w
  int count;
};

template <int GS, int WAVES>
__global__ void __launch_bounds__(WAVES * 64)
    qmm_group_kernel(const uint16_t* __restrict__ X, int64_t ldx, const float* __restrict__ XS, GroupArgs a, int M,
                     int KG, int BM, int f32) {
  extern __shared__ float lds[];
  int w = 0;
#pragma unroll
  for (int i = 1; i < GROUP_MAX; ++i)
    if (i < a.count && (int)blockIdx.x >= a.first[i]) w = i;
  if ((int)blockIdx.z >= a.sk[w]) return;
  qmm_block<GS, WAVES>(X, ldx, XS, a.w[w], a.s[w], a.b[w], a.sb_stride[w], a.out[w], a.part[w], M, a.n[w], KG, a.sk[w],
                       BM, f32, blockIdx.x - a.first[w], blockIdx.z, lds);
}

// The grouped launch in the one-launch form (see qmm_fat_block): every weight's K split is 4, 8 or 16.
// the grouped launch whose slices are added up by the last workgroup of a tile to finish (qmm_arrive_kernel's way);
// a weight whose K is not split stores its rows itself
template <int GS, int WAVES>
__global__ void __launch_bounds__(WAVES * 64)
    qmm_group_arrive_kernel(const uint16_t* __restrict__ X, int64_t ldx, const float* __restrict__ XS, GroupArgs a, int M,
                            int KG, int BM, int f32) {
  extern __shared__ float lds[];
  __shared__ int last;
  int w = 0;
#pragma unroll
  for (int i = 1; i < GROUP_MAX; ++i)
    if (i < a.count && (int)blockIdx.x >= a.first[i]) w = i;
  if ((int)blockIdx.z >= a.sk[w]) return;
  const int block = blockIdx.x - a.first[w];
  qmm_block<GS, WAVES, true>(X, ldx, XS, a.w[w], a.s[w], a.b[w], a.sb_stride[w], a.out[w], a.part[w], M, a.n[w], KG,
                             a.sk[w], BM, f32, block, blockIdx.z, lds);
  if (a.sk[w] > 1)
    qmm_arrive_tail<WAVES>(a.counters[w] + (size_t)block * TF_QMM_COUNTER_STRIDE, a.part[w], a.out[w], M, a.n[w],
                           a.sk[w], BM, f32, block, &last);
}

template <int GS>
__global__ void __launch_bounds__(1024)
    qmm_group_fat_kernel(const uint16_t* __restrict__ X, int64_t ldx, const float* __restrict__ XS, GroupArgs a, int M,
                         int KG, int BM, int f32) {
  extern __shared__ float lds[];
  int w = 0;
#pragma unroll
  for (int i = 1; i < GROUP_MAX; ++i)
    if (i < a.count && (int)blockIdx.x >= a.first[i]) w = i;
  qmm_fat_block<GS, 16>(X, ldx, XS, a.w[w], a.s[w], a.b[w], a.sb_stride[w], a.out[w], M, a.n[w], KG, a.sk[w], BM, f32,
                        blockIdx.x - a.first[w], lds);
}

// p[0] + p[stride] + ... (n terms, in that order); eight loads go out together before they are added
__device__ __forceinline__ float ordered_sum(const float* __restrict__ p, long long stride, int n) {
  float acc = 0.f;
  for (int s0 = 0; s0 < n; s0 += 8) {
    float v[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = p[(long long)(s0 + j < n ? s0 + j : n - 1) * stride];
#pragma unroll
    for (int j = 0; j < 8; ++j)
      if (s0 + j < n) acc = s0 + j ? acc + v[j] : v[j];
  }
  return acc;
}

__global__ void qmm_group_reduce_kernel(GroupArgs a, int M, int f32) {
  int w = 0;
#pragma unroll
  for (int i = 1; i < GROUP_MAX; ++i)
    if (i < a.count && (int)blockIdx.x >= a.first[i]) w = i;
  if (a.sk[w] == 1) return;
  const long long total = (long long)M * a.n[w];
  const long long i = (long long)(blockIdx.x - a.first[w]) * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const float* part = a.part[w];
  const float acc = ordered_sum(part + i, total, a.sk[w]);
  if (f32) reinterpret_cast<float*>(a.out[w])[i] = acc;
  else reinterpret_cast<uint16_t*>(a.out[w])[i] = (uint16_t)f32_bf16_bits(acc);
}

// the K slices' partial sums added in slice order, then rounded once (qmm.cu:222-230)
__global__ void qmm_reduce_kernel(const float* __restrict__ part, void* __restrict__ out, long long total, int SK,
                                  int f32) {
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const float acc = ordered_sum(part + i, total, SK);
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
constexpr int FAT_ROWS = 8;          // rows up to which tf_qmm runs the one-launch form
constexpr int ARRIVE_ROWS = QRB;      // rows up to which, given arrival counters, the split launch adds its own slices

// Waves a workgroup of the expert GEMV: few workgroups (a small batch) spread each one's K over 16 waves, many
// workgroups keep 4 longer-running waves each so that more of them are resident.  Scheduling only: bits do not move.
int expert_waves(int64_t grid) { return grid < 384 ? 16 : grid < 768 ? 8 : 4; }

template <int GS, int NM, int EPI>
int launch_experts(const uint16_t* x, int64_t x_stride, int slots, const uint32_t* w, int kg, int nb, const int* items,
                   const int* counts, const int* members, void* out, int n, float limit, int64_t max_units,
                   hipStream_t stream) {
  const int nb2 = (nb + 1) / 2;
  const int64_t max_items = (max_units + nb - 1) / nb;
  const int64_t grid = max_items * nb2;
  if (grid < 1) return 0;
  TF_REQUIRE(grid <= 0x7FFFFFFF, "experts: %lld workgroups exceed the grid limit", (long long)grid);
  const size_t smem = sizeof(float) * expert_lds_floats(NM);
  TF_REQUIRE(smem <= 64 * 1024, "experts: K/gs = %d groups need %zu bytes of LDS (limit 65536)", kg, smem);
  const dim3 g((unsigned)grid, 16 / RBMAX);          // decode items hold at most 16 pairs
#define TF_GO(W_)                                                                                                  \
  expert_kernel<GS, NM, EPI, W_><<<g, W_ * 64, smem, stream>>>(x, x_stride, slots, w, kg, nb, items, counts, members, \
                                                               out, n, limit)
  switch (expert_waves(grid)) {
    case 16: TF_GO(16); break;
    case 8: TF_GO(8); break;
    default: TF_GO(4);
  }
#undef TF_GO
  TF_LAUNCH_OK("tf_experts_run");
  return 0;
}

template <int GS, int NM, int EPI>
int launch_experts_desc(const uint16_t* x, int64_t x_stride, int slots, const uint32_t* w, int kg, int nb,
                        const int* desc, const int* counts, void* out, int n, float limit, int64_t max_items,
                        hipStream_t stream) {
  const int nb2 = (nb + 1) / 2;
  const int64_t grid = max_items * nb2;
  if (grid < 1) return 0;
  TF_REQUIRE(grid <= 0x7FFFFFFF, "experts: %lld workgroups exceed the grid limit", (long long)grid);
  const size_t smem = sizeof(float) * expert_lds_floats(NM);
  const dim3 g((unsigned)grid);
#define TF_GO(W_)                                                                                                 \
  expert_desc_kernel<GS, NM, EPI, W_><<<g, W_ * 64, smem, stream>>>(x, x_stride, slots, w, kg, nb, desc, counts, out, n, \
                                                                    limit)
  switch (expert_waves(grid)) {
    case 16: TF_GO(16); break;
    case 8: TF_GO(8); break;
    default: TF_GO(4);
  }
#undef TF_GO
  TF_LAUNCH_OK("tf_experts_run_desc");
  return 0;
}

}  // namespace
}  // namespace tf

using namespace tf;

extern "C" int tf_experts_run_desc(int gs, int epi, const uint16_t* x, int64_t x_stride, int slots, const uint32_t* w,
                                   int kg, int nb, const int32_t* desc, const int32_t* counts, void* out, int n,
                                   float limit, int64_t max_items, tf_stream_t stream) {
  clear_error();
  TF_REQUIRE(gs == 32 || gs == 64, "experts: groups of 32 or 64 inputs, not %d", gs);
  TF_REQUIRE(x && w && desc && counts && out, "experts: null pointer argument");
  TF_REQUIRE(kg >= 1 && nb >= 1 && n == nb * 32, "experts: n (%d) must be the column blocks (%d) times 32", n, nb);
  TF_REQUIRE(aligned16(x) && x_stride % 8 == 0, "x: rows of K = groups * group size inputs, 16-byte aligned");
  TF_REQUIRE(aligned16(w), "w must be 16-byte aligned");
  TF_REQUIRE(slots >= 0 && max_items >= 0, "experts: negative slots or max_items");
  hipStream_t s = as_stream(stream);
#define TF_RUN(GS_, NM_, EPI_)            \
  if (gs == GS_ && epi == EPI_)           \
    return launch_experts_desc<GS_, NM_, EPI_>(x, x_stride, slots, w, kg, nb, desc, counts, out, n, limit, max_items, s);
  TF_RUN(32, 1, 0) TF_RUN(32, 1, 1) TF_RUN(32, 2, 2) TF_RUN(64, 1, 0) TF_RUN(64, 1, 1) TF_RUN(64, 2, 2)
#undef TF_RUN
  set_error("experts: no kernel for group %d and epilogue %d", gs, epi);
  return 1;
}

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
#define TF_RUN(GS_, NM_, EPI_)                                                                                    \
  if (gs == GS_ && epi == EPI_)                                                                                   \
    return launch_experts<GS_, NM_, EPI_>(x, x_stride, slots, w, kg, nb, items, counts, members, out, n, limit, \
                                          max_units, s);
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

// tf_qmm and tf_qmm_static: the checks and launches of the decode-form matmul; `part` holds the K slices.
static int qmm_launch(const uint16_t* x, int64_t ldx, const float* xs, const uint32_t* weight, const uint16_t* scales,
                      const uint16_t* biases, int64_t sb_stride, void* out, float* part, int32_t* counters,
                      int n_counters, int m, int n, int k, int sk, int gs, int bm, int f32, int reduce,
                      tf_stream_t stream) {
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
  const size_t smem = sizeof(float) * ((size_t)QMM_WAVES * QRB * 64);
  TF_REQUIRE((int64_t)tiles * rts <= 0x7FFFFFFF && sk <= 65535, "qmm: grid too large");
  const int64_t fat_blocks = (int64_t)((n + 63) / 64) * ((m + RBMAX - 1) / RBMAX);
  const dim3 grid((unsigned)(tiles * rts), 1, (unsigned)sk);
  if (reduce && sk > 1 && counters && m <= ARRIVE_ROWS && (int64_t)tiles * rts <= n_counters) {
    // one pass of rows, and arrival counters: the slices are added up by the last workgroup of a tile to finish.
    // Hundreds of four-wave workgroups beat the one-launch form's workgroup a column tile and row pair: 4096 x 4096
    // 6.0 us at 1 row against 7.5, 7.1 at 4 against 8.5 (9.1 against 8.3 at 8, the one shape where that form wins);
    // 5120 x 17408 at 8 rows 24 against 40
    if (gs == 64)
      qmm_arrive_kernel<64, QMM_WAVES><<<grid, QMM_WAVES * 64, smem, s>>>(x, ldx, xs, weight, scales, biases, sb_stride,
                                                                           out, part, counters, m, n, kg, sk, bm, f32);
    else
      qmm_arrive_kernel<32, QMM_WAVES><<<grid, QMM_WAVES * 64, smem, s>>>(x, ldx, xs, weight, scales, biases, sb_stride,
                                                                           out, part, counters, m, n, kg, sk, bm, f32);
    TF_LAUNCH_OK("tf_qmm");
    return 0;
  }
  if (reduce && (m <= RBMAX || (m <= FAT_ROWS && fat_blocks <= 512)) && (sk == 2 || sk == 4 || sk == 8 || sk == 16)) {
    // few rows: split and reduce in one launch, a workgroup of 8 or 16 waves taking every slice of a tile for RBMAX
    // rows in one pass (same bits), while those workgroups fit the chip at once (512 of 16 waves).  Past that, and
    // with many rows, the split launch is better: its waves keep their one or two groups in registers from pass to
    // pass.
    bm = RBMAX;
    const dim3 fat((unsigned)(tiles * ((m + RBMAX - 1) / RBMAX)));
    const size_t fat_smem = sizeof(float) * ((size_t)4 * sk * RBMAX * 64);
#define TF_FAT(GS_, FW_) \
  qmm_fat_kernel<GS_, FW_><<<fat, FW_ * 64, fat_smem, s>>>(x, ldx, xs, weight, scales, biases, sb_stride, out, m, n, kg, sk, bm, f32)
    if (gs == 64) {
      if (sk == 2) TF_FAT(64, 8);
      else TF_FAT(64, 16);
    } else {
      if (sk == 2) TF_FAT(32, 8);
      else TF_FAT(32, 16);
    }
#undef TF_FAT
    TF_LAUNCH_OK("tf_qmm");
    return 0;
  }
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

extern "C" int tf_qmm(const uint16_t* x, int64_t ldx, const float* xs, const uint32_t* weight, const uint16_t* scales,
                      const uint16_t* biases, int64_t sb_stride, void* out, float* part, int32_t* counters,
                      int n_counters, int m, int n, int k, int sk, int gs, int bm, int f32, int reduce,
                      tf_stream_t stream) {
  clear_error();
  TF_REQUIRE(!counters || n_counters >= 0, "qmm: a negative number of counters");
  return qmm_launch(x, ldx, xs, weight, scales, biases, sb_stride, out, part, counters, n_counters, m, n, k, sk, gs, bm,
                    f32, reduce, stream);
}

// The K slices of tf_qmm_static: one array a GPU, part of the loaded code object, so no call ever allocates it.
// Host code may not use the array's name as an address; it asks the runtime once a device for where that device
// holds its copy and passes that pointer to the kernels like any other buffer.
static __device__ __align__(256) float scratch[TF_QMM_STATIC_FLOATS];
// the arrival counters of the column tiles, zero when the image is loaded and put back to zero by every launch
static __device__ __align__(256) int scratch_counters[TF_QMM_STATIC_COUNTERS * TF_QMM_COUNTER_STRIDE];

// where the current device holds the two arrays (asked once a device)
static bool static_scratch(float** part, int32_t** counters) {
  constexpr int MAX_DEVICES = 64;
  static float* where[MAX_DEVICES];
  static int32_t* where_counters[MAX_DEVICES];
  static std::mutex guard;
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) {
    set_error("tf_qmm_static: no current HIP device (or its index is %d or more)", MAX_DEVICES);
    return false;
  }
  std::lock_guard<std::mutex> lock(guard);
  if (!where[dev]) {
    void *p = nullptr, *c = nullptr;
    hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e == hipSuccess) e = hipGetSymbolAddress(&c, HIP_SYMBOL(scratch_counters));
    if (e != hipSuccess || !p || !c) {
      set_error("tf_qmm_static: hipGetSymbolAddress failed on device %d: %s", dev, hipGetErrorString(e));
      return false;
    }
    where[dev] = static_cast<float*>(p);
    where_counters[dev] = static_cast<int32_t*>(c);
  }
  *part = where[dev];
  *counters = where_counters[dev];
  return true;
}

extern "C" int tf_qmm_static(const uint16_t* x, int64_t ldx, const float* xs, const uint32_t* weight,
                             const uint16_t* scales, const uint16_t* biases, int64_t sb_stride, void* out, int m, int n,
                             int k, int sk, int gs, int bm, int f32, tf_stream_t stream) {
  clear_error();
  TF_REQUIRE(m >= 1 && n >= 1 && sk >= 1, "qmm: null pointer or empty shape");
  TF_REQUIRE(sk == 1 || (int64_t)sk * m * n <= (int64_t)TF_QMM_STATIC_FLOATS,
             "tf_qmm_static: %d slices x %d rows x %d columns = %lld fp32 partial sums exceed the built-in %lld; use "
             "tf_qmm with a part buffer", sk, m, n, (long long)sk * m * n, (long long)TF_QMM_STATIC_FLOATS);
  float* part = nullptr;
  int32_t* counters = nullptr;
  if (sk > 1 && !static_scratch(&part, &counters)) return 1;
  return qmm_launch(x, ldx, xs, weight, scales, biases, sb_stride, out, part, counters, TF_QMM_STATIC_COUNTERS, m, n, k,
                    sk, gs, bm, f32, 1, stream);
}

extern "C" int tf_qmm_group(const uint16_t* x, int64_t ldx, const float* xs, int count, const uint32_t* const* weights,
                            const uint16_t* const* scales, const uint16_t* const* biases, const int64_t* sb_strides,
                            void* const* outs, float* const* parts, int32_t* const* counters, const int* n_counters,
                            const int* ns, const int* sks, int m, int k, int gs, int bm, int f32, tf_stream_t stream) {
  clear_error();
  TF_REQUIRE(gs == 32 || gs == 64, "groups of 32 or 64");
  TF_REQUIRE(bm == 16 || bm == 32 || bm == 64, "row tile 16, 32 or 64");
  TF_REQUIRE(count >= 1 && count <= GROUP_MAX, "qmm_group: 1 to %d weights, not %d", GROUP_MAX, count);
  TF_REQUIRE(!counters || n_counters, "qmm_group: counters come with their counts");
  TF_REQUIRE(x && xs && weights && scales && biases && sb_strides && outs && parts && ns && sks && m >= 1,
             "qmm_group: null pointer or empty shape");
  TF_REQUIRE(aligned16(x) && (m == 1 || ldx % 8 == 0), "x rows must start on 16-byte boundaries");
  TF_REQUIRE(ldx >= k || m == 1, "x: (M, K) bf16 with contiguous rows");
  TF_REQUIRE(k % gs == 0, "K splits into whole groups a slice");
  const int kg = k / gs;
  // one pass of rows and every split weight's arrival counters: the arriving form, as tf_qmm
  bool arrive = counters && m <= ARRIVE_ROWS;
  for (int i = 0; i < count && arrive; ++i)
    arrive = ns && sks && (sks[i] == 1 || (counters[i] && (ns[i] + 63) / 64 * ((m + bm - 1) / bm) <= n_counters[i]));
  // few rows and every K split 4, 8 or 16: the one-launch form (two rows a workgroup), as tf_qmm
  bool fat = !arrive && m <= FAT_ROWS;
  int64_t fat_blocks = 0;
  for (int i = 0; i < count && fat; ++i) {
    fat = ns && sks && ns[i] >= 1 && (sks[i] == 4 || sks[i] == 8 || sks[i] == 16);
    if (fat) fat_blocks += (int64_t)((ns[i] + 63) / 64) * ((m + RBMAX - 1) / RBMAX);
  }
  fat = fat && (m <= RBMAX || fat_blocks <= 512);
  if (fat) bm = RBMAX;
  const int rts = (m + bm - 1) / bm;
  GroupArgs a{}, r{};
  int max_sk = 1;
  int64_t blocks = 0, chunks = 0;
  bool any_split = false;
  for (int i = 0; i < count; ++i) {
    const int n = ns[i], sk = sks[i], npad = (n + 127) / 128 * 128;
    TF_REQUIRE(weights[i] && scales[i] && biases[i] && outs[i] && n >= 1, "qmm_group: null pointer or empty shape");
    TF_REQUIRE(sk >= 1 && sk <= 65535 && kg % sk == 0, "K splits into whole groups a slice");
    TF_REQUIRE(sb_strides[i] >= npad, "scales and biases: (K / gs, n padded to 128) bf16, rows may be strided");
    TF_REQUIRE(aligned16(weights[i]), "packed weight must be 16-byte aligned");
    TF_REQUIRE(sk == 1 || parts[i], "part: at least (SK, M, n) fp32 is needed when K is split");
    a.w[i] = weights[i];
    a.s[i] = scales[i];
    a.b[i] = biases[i];
    a.out[i] = outs[i];
    a.part[i] = parts[i];
    a.counters[i] = arrive ? counters[i] : nullptr;
    a.sb_stride[i] = sb_strides[i];
    a.n[i] = n;
    a.sk[i] = sk;
    a.first[i] = (int)blocks;
    r.first[i] = (int)chunks;
    blocks += (int64_t)((n + 63) / 64) * rts;
    chunks += ((int64_t)m * n + 255) / 256;
    TF_REQUIRE(blocks <= 0x7FFFFFFF && chunks <= 0x7FFFFFFF, "qmm_group: grid too large");
    max_sk = sk > max_sk ? sk : max_sk;
    any_split = any_split || sk > 1;
  }
  a.count = count;
  a.first[count] = (int)blocks;
  hipStream_t s = as_stream(stream);
  if (fat) {
    const size_t fat_smem = sizeof(float) * ((size_t)4 * max_sk * RBMAX * 64);
    if (gs == 64) qmm_group_fat_kernel<64><<<(unsigned)blocks, 1024, fat_smem, s>>>(x, ldx, xs, a, m, kg, bm, f32);
    else qmm_group_fat_kernel<32><<<(unsigned)blocks, 1024, fat_smem, s>>>(x, ldx, xs, a, m, kg, bm, f32);
    TF_LAUNCH_OK("tf_qmm_group");
    return 0;
  }
  const size_t smem = sizeof(float) * ((size_t)QMM_WAVES * QRB * 64);
  const dim3 grid((unsigned)blocks, 1, (unsigned)max_sk);
  if (arrive) {
    if (gs == 64) qmm_group_arrive_kernel<64, QMM_WAVES><<<grid, QMM_WAVES * 64, smem, s>>>(x, ldx, xs, a, m, kg, bm, f32);
    else qmm_group_arrive_kernel<32, QMM_WAVES><<<grid, QMM_WAVES * 64, smem, s>>>(x, ldx, xs, a, m, kg, bm, f32);
    TF_LAUNCH_OK("tf_qmm_group");
    return 0;
  }
  if (gs == 64) qmm_group_kernel<64, QMM_WAVES><<<grid, QMM_WAVES * 64, smem, s>>>(x, ldx, xs, a, m, kg, bm, f32);
  else qmm_group_kernel<32, QMM_WAVES><<<grid, QMM_WAVES * 64, smem, s>>>(x, ldx, xs, a, m, kg, bm, f32);
  TF_LAUNCH_OK("tf_qmm_group");
  if (any_split) {
    int first[GROUP_MAX + 1];
    for (int i = 0; i < count; ++i) first[i] = r.first[i];
    r = a;
    for (int i = 0; i < count; ++i) r.first[i] = first[i];
    r.first[count] = (int)chunks;
    qmm_group_reduce_kernel<<<(unsigned)chunks, 256, 0, s>>>(r, m, f32);
    TF_LAUNCH_OK("tf_qmm_group reduce");
  }
  return 0;
}
