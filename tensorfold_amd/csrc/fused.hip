// The decode MoE layer's experts in ONE launch: up projection (+ activation), down projection and the weighted
// combine, so that the layer's weights stream from HBM as one run instead of three launches with their ramps.
//
// Workgroups [0, U) take the up units (item, 64 columns of NI); workgroups [U, U + D) take the down units (item,
// 64 columns of D).  A down unit first requests its weights, then waits until all the up units of its item have
// published the item's activations (an arrival counter an item), then multiplies.  The hardware hands workgroups
// out in index order, so every up unit is running or done before a down unit can occupy a slot: the wait cannot
// deadlock; it is bounded anyway, and a timeout raises a status flag and abandons the unit.  The last down unit to
// finish a (token, 64 columns) cell adds the token's slots in slot order (fp32, as tf_moe_combine) and writes bf16.
//
// The chip's eight XCDs have separate L2s.  What one workgroup hands to another (activations, their group sums, the
// pair outputs) is written and read with agent-scope relaxed accesses, which are coherent by themselves; a
// producer waits for its stores to be acknowledged before it bumps the counter.  No cache-wide write-back or
// invalidate is ever issued (they cost about half a microsecond of an XCD's L2 each).  No float atomics: every sum
// has a fixed order, and the bits equal those of tf_experts_run (up), tf_experts_run (down) and tf_moe_combine run
// one after the other.

#include "gemv.h"
#include "routing.h"

namespace tf {
namespace {

// Waves a workgroup from a launch's size (measured on config 1): few workgroups want many waves each to keep enough
// loads in flight; past about 1,300 workgroups of the routing launch (about 1,700 of the down launch) eight waves
// each no longer fit the chip at once and four are faster.
int fused_waves(int64_t grid) { return grid < 768 ? 16 : grid < 2560 ? 8 : 4; }
// the same for the one-launch layer cut along the intermediate width, whose units stream an up and a down part
int sliced_waves(int64_t grid) { return grid < 384 ? 16 : grid < 1280 ? 8 : 4; }

// An item's arrival counter sits alone in 256 bytes.  The 42 down units of an item poll it, and with the counters of
// all items side by side (two cache lines for 48 items) a thousand polling workgroups queued on one memory channel,
// behind which every workgroup's weight stream waited in turn: the launch took 75 us instead of 46 (config 1, 8 tokens).
constexpr int DONE_STRIDE = TF_DONE_STRIDE;

struct WaitItem {
  const int* flag;
  int want;
  int spins;
  int* status;
  __device__ __forceinline__ bool operator()() const {
    __shared__ int ok;
    if (threadIdx.x == 0) {
      int left = spins, seen = 0;
      while ((seen = __hip_atomic_load(flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) < want && --left > 0)
        __builtin_amdgcn_s_sleep(2);
      ok = seen >= want;
      if (!ok) atomicExch(status, 1);
    }
    __syncthreads();
    return ok != 0;
  }
};

// Ints between the arrival counters of two (token, 64 columns) cells: with few rows each counter sits alone in 64
// bytes (at one token the 252 units of a launch arrive within a microsecond on 42 counters).
int arrive_stride(int rows) { return rows <= 64 ? TF_ARRIVE_STRIDE : 1; }

// A down unit has written its 64 columns of y (agent-scope stores) for its rows: count it in each row's token; the
// unit that completes a (token, 64 columns) cell adds the token's slots in slot order (fp32 fma, as tf_moe_combine)
// and writes bf16.  `arrive` [tokens * NB2d * astride] starts at zero and is left at zero.
template <int WAVES>
__device__ __forceinline__ void combine_cells(const int* pairs, int cnt, int slots, int cb2, int NB2d, int D, int astride,
                                              const float* __restrict__ wts, const float* __restrict__ y,
                                              uint16_t* __restrict__ out, int* __restrict__ arrive) {
  __builtin_amdgcn_s_waitcnt(0);      // every store of this wave is acknowledged ...
  __syncthreads();                    // ... of every wave ...
  // ... then wave r counts the unit in for its row r and, if that completes the cell, sums it; the other waves
  // are done (an item has at most as many rows as a workgroup has waves)
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int col = cb2 * 64 + lane;
  for (int r = wave; r < cnt; r += WAVES) {
    const int token = pairs[r] / slots;
    int done = 0;
    if (lane == 0) {
      int* cell = arrive + ((size_t)token * NB2d + cb2) * astride;
      done = __hip_atomic_fetch_add(cell, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == slots - 1;
      if (done) __hip_atomic_store(cell, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // every unit has arrived: ready for the next launch
    }
    if (!__builtin_amdgcn_readfirstlane(done) || col >= D) continue;
    float a = 0.f;
    // eight slots' loads go out together (one trip to memory instead of eight), then the sum in slot order
    for (int k0 = 0; k0 < slots; k0 += 8) {
      float v[8], w[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int k = k0 + j < slots ? k0 + j : slots - 1;
        w[j] = wts[(size_t)token * slots + k];
        v[j] = ld_agent(y + ((size_t)token * slots + k) * D + col);
      }
#pragma unroll
      for (int j = 0; j < 8; ++j)
        if (k0 + j < slots) a = fmaf(w[j], v[j], a);
    }
    out[(size_t)token * D + col] = (uint16_t)f32_bf16_bits(a);
  }
}

// The down projection from item descriptors with the combine folded in (see combine_cells).
template <int GS, int WAVES>
__global__ void __launch_bounds__(WAVES * 64)
    down_combine_kernel(const uint16_t* __restrict__ act, int slots, const uint32_t* __restrict__ Wdown, int D, int NI,
                        const int* __restrict__ desc, const float* __restrict__ wts, float* __restrict__ y, uint16_t* __restrict__ out, int* __restrict__ arrive, int astride) {
  extern __shared__ float lds[];
  __shared__ int pairs[16];
  TF_MARK(0);
  __builtin_amdgcn_s_setprio(3);       // the descriptor and the first requests issue ahead of the workgroups that already stream
  const int NB = D / 32, NB2d = (NB + 1) >> 1;
  const int it = blockIdx.x / NB2d, cb2 = blockIdx.x - it * NB2d;
  // the descriptor's words are requested with the count, not after it (a row past the count exists and is ignored)
  const int* d = desc + (size_t)(1 + it) * DESC;
  const int n_items = desc[0], e = d[0], cnt = d[1], p0 = d[4], p1 = d[5];
  if (it >= n_items) return;
  if (threadIdx.x < DTILE) pairs[threadIdx.x] = threadIdx.x ? p1 : p0;
  __syncthreads();
  NoHook none;
  expert_unit<GS, 1, 0, WAVES, COH_OUT>(act, NI, 0, Wdown, NI / GS, NB, e, cnt, pairs, cb2, y, D, 0.f, lds, none);
  combine_cells<WAVES>(pairs, cnt, slots, cb2, NB2d, D, astride, wts, y, out, arrive);
  TF_MARK(5);
}

template <int GS, int NM, int EPI_UP, int WAVES>
__global__ void __launch_bounds__(WAVES * 64)
    moe_fused_kernel(const uint16_t* __restrict__ X, int64_t x_stride, int slots, const uint32_t* __restrict__ Wup,
                     const uint32_t* __restrict__ Wdown, int D, int NI, const int* __restrict__ desc,
                     const int* __restrict__ counts, const float* __restrict__ wts, uint16_t* __restrict__ act,
                     float* __restrict__ y,
                     uint16_t* __restrict__ out, int* __restrict__ done, int* __restrict__ arrive,
                     int* __restrict__ status, float limit, int max_items, int spins, int astride) {
  extern __shared__ float lds[];
  __shared__ int pairs[16];
  const int NB2u = (NI / 32 + 1) >> 1, NB2d = (D / 32 + 1) >> 1;
  const int U = max_items * NB2u;
  const int b = blockIdx.x, tid = threadIdx.x;
  const bool up = b < U;
  const int it = up ? b / NB2u : (b - U) / NB2d;
  const int cb2 = up ? b - it * NB2u : (b - U) - it * NB2d;
  // the descriptor's words are requested with the count, not after it (a row past the count exists and is ignored)
  const int* d = desc + (size_t)(1 + it) * DESC;
  const int n_items = desc[0], e = d[0], cnt = d[1], p0 = d[4], p1 = d[5];
  if (it >= n_items) return;
  if (tid < DTILE) pairs[tid] = tid ? p1 : p0;
  __syncthreads();
  if (up) {
    NoHook none;
    expert_unit<GS, NM, EPI_UP, WAVES, COH_OUT>(X, x_stride, slots, Wup, D / GS, NI / 32, e, cnt, pairs, cb2, act, NI,
                                                limit, lds, none);
    __builtin_amdgcn_s_waitcnt(0);      // every store of this wave is acknowledged ...
    __syncthreads();                    // ... of every wave ...
    if (tid == 0) __hip_atomic_fetch_add(done + (size_t)it * DONE_STRIDE, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // ... then it counts
    return;
  }
  WaitItem wait{done + (size_t)it * DONE_STRIDE, NB2u, spins, status};
  constexpr int DCOH = COH_IN | COH_OUT;
  if (!expert_unit<GS, 1, 0, WAVES, DCOH>(act, NI, 0, Wdown, NI / GS, D / 32, e, cnt, pairs, cb2, y, D, 0.f, lds, wait))
    return;                     // the wait ran out: status is set, nothing is published
  combine_cells<WAVES>(pairs, cnt, slots, cb2, NB2d, D, astride, wts, y, out, arrive);
}


// ---- the whole layer in one launch, cut along the intermediate width --------------------------------------------------
//
// A unit = (item of one or two pairs, 64 columns of NI).  It runs the up unit as route_up_kernel does, keeps the 64
// activations of its rows in LDS, and goes straight on to the part of the down projection those activations feed:
// one group of inputs (two at groups of 32) of all of the expert's D columns, whose weights depend on nothing the
// unit computes and are on their way before its up projection has been summed.  What it leaves is each group's term
// t = fma(xs, b, P s) for every column of D: fp32 `part` [pair][64 columns of D][group][64], written through to
// memory.  The unit that brings a (pair, 64 columns of D) cell its last group adds the terms up in the order the down
// launch adds them (the groups of a K slice in turn, then the slices: gemv_stream with SEPG) and stores the pair's
// output; the one that then completes a (token, 64 columns) cell adds the token's slots in slot order and writes
// bf16: the bits of tf_moe_route_up + tf_moe_down_combine.  Nobody waits for anybody.
//
// Hand-offs are the last-arriver scheme of combine_cells.  To spread the adding-up over the units of an item instead
// of leaving it all to whichever ends last, a unit starts its walk over the D columns at a place of its own and counts
// each 64 columns in as it goes: the count for the columns of step k - 2 is issued at step k, after the wave has
// waited for step k's weights, which it requested after the stores of step k - 2 (vector memory operations of a wave
// complete in the order they were issued, so those stores have been acknowledged).

struct SliceArgs {
  const uint32_t* Wdown;
  float* part;          // [pairs][D / 64][NI / gs][64]
  float* y;             // [pairs][D]
  uint16_t* out;        // [rows][D]
  int* c1;              // arrival counts a (pair, 64 columns of D), TF_ARRIVE_STRIDE ints apart, zero between launches
  int* c2;              // arrival counts a (token, 64 columns of D), likewise
  const float* wts;     // the pairs' weights when the picks were given (no logits)
};

// The unit's inputs of one (64 columns of D): 64 / GS groups of one matrix.
template <int GS>
struct DownStage {
  Stage<GS, 1> g[64 / GS];
};

// A wave's walk over the 64-column blocks of D: step k takes block (rot + wave + WAVES k) mod NBD2.
template <int GS, int WAVES>
struct DownWalk {
  static constexpr int G1 = 64 / GS, BW = block_words(GS);
  const uint32_t* wexp;        // the expert's down matrix
  int NBd, NBD2, KGd, g0, ng, rot, wave, lane, n;
  __device__ __forceinline__ int db(int k) const {
    const int q = rot + wave + WAVES * k;
    return q >= NBD2 ? q - NBD2 : q;
  }
  __device__ __forceinline__ bool col_ok(int k) const { return 2 * db(k) + (lane >> 5) < NBd; }
  __device__ __forceinline__ void load(DownStage<GS>& s, int k) const {
    const int nb = min(2 * db(k) + (lane >> 5), NBd - 1), c = lane & 31;
    const uint32_t* blk = wexp + ((size_t)nb * KGd + g0) * BW;
#pragma unroll
    for (int gi = 0; gi < G1; ++gi) {
      const uint32_t* b = blk + (size_t)(gi < ng ? gi : 0) * BW;
#pragma unroll
      for (int i = 0; i < GS / 32; ++i) s.g[gi].w[0][i] = ldg16(b + i * 128 + c * 4);
      s.g[gi].s[0] = s.g[gi].b[0] = __builtin_nontemporal_load(b + 32 * GS / 8 + c);
    }
  }
};

// The terms of one step: t[r][gi] = fma(xs, b, P s) of row r and group gi for the lane's column.
template <int GS, int RB>
__device__ __forceinline__ void down_terms(const DownStage<GS>& s, const float (&sc)[RB][64 / GS],
                                           float (&t)[RB][64 / GS]) {
#pragma unroll
  for (int gi = 0; gi < 64 / GS; ++gi) {
    float p[1][RB];
#pragma unroll
    for (int r = 0; r < RB; ++r) p[0][r] = 0.f;
#pragma unroll
    for (int i = 0; i < GS / 32; ++i) chunk_dot<GS, 1, RB>(p, s.g[gi], i);
#pragma unroll
    for (int r = 0; r < RB; ++r) asm volatile("s_nop 2" : "+v"(p[0][r]));
#pragma unroll
    for (int r = 0; r < RB; ++r) {
      const float pq = fmaf(-128.f, sc[r][gi], p[0][r]);
      const float scale = __uint_as_float(s.g[gi].s[0] << 16);
      const float bias = __uint_as_float(s.g[gi].b[0] & 0xFFFF0000u);
      t[r][gi] = group_term(pq, scale, sc[r][gi], bias);
    }
  }
}

// The groups' terms of one (pair, 64 columns) cell added up as the down launch adds them: the groups of a K slice in
// turn from zero, then the slices in slice order.  src: the cell's terms [KG][64], already offset by the lane.
__device__ __forceinline__ float slice_tree(const float* src, int KG) {
  float total = 0.f, sacc = 0.f;
  bool first = true;
  int q = 0;
  while (q < SLICES && slice_begin(q + 1, KG) == slice_begin(q, KG)) ++q;
  int end = q < SLICES ? slice_begin(q + 1, KG) : -1;
  for (int g0 = 0; g0 < KG; g0 += 16) {
    float v[16];
#pragma unroll
    for (int j = 0; j < 16; ++j) v[j] = ld_agent(src + (size_t)min(g0 + j, KG - 1) * 64);
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      if (g0 + j >= KG) break;
      sacc = __fadd_rn(sacc, v[j]);
      if (g0 + j + 1 == end) {
        total = first ? sacc : __fadd_rn(total, sacc);
        first = false;
        sacc = 0.f;
        ++q;
        while (q < SLICES && slice_begin(q + 1, KG) == slice_begin(q, KG)) ++q;
        end = q < SLICES ? slice_begin(q + 1, KG) : -1;
      }
    }
  }
  return total;
}

// A unit's second half: every wave walks its share of D's 64-column blocks.
template <int GS, int WAVES, int RB>
__device__ __forceinline__ void down_slices(const DownWalk<GS, WAVES>& walk, DownStage<GS> (&st)[DEPTH], const int* pairs,
                                            const uint32_t* actw, int slots, int D, int NU, const SliceArgs& sa,
                                            const float* __restrict__ L, int64_t ldl, int NE, int TOPK, int shared) {
  constexpr int G1 = 64 / GS, CH = GS / 32;
  const int lane = walk.lane, n = walk.n, KG = walk.KGd, NBD2 = walk.NBD2;
  int pr[RB];
#pragma unroll
  for (int r = 0; r < RB; ++r) pr[r] = pairs[r];
  const int pr_lane = lane == 0 ? pr[0] : pr[RB - 1];
  // the rows' 64 activations as the dot products want them, and their sums a group
  float sc[RB][G1];
#pragma unroll
  for (int d = 0; d < DEPTH; ++d)
#pragma unroll
    for (int gi = 0; gi < G1; ++gi)
#pragma unroll
      for (int r = 0; r < RB; ++r)
#pragma unroll
        for (int i = 0; i < CH; ++i) st[d].g[gi].x[r][i] = actw[r * 32 + (gi * CH + i) * 16 + (lane & 15)];
#pragma unroll
  for (int r = 0; r < RB; ++r)
#pragma unroll
    for (int gi = 0; gi < G1; ++gi) sc[r][gi] = stage_row_sum<GS, 1>(st[0].g[gi], r);

  auto bump = [&](int k) {
    int v = 0;
    if (lane < RB)
      v = __hip_atomic_fetch_add(sa.c1 + ((size_t)pr_lane * NBD2 + walk.db(k)) * TF_ARRIVE_STRIDE, 1, __ATOMIC_RELAXED,
                                 __HIP_MEMORY_SCOPE_AGENT);
    return v;
  };
  // bit RB k + r of `mine`: this wave's count completed the cell (pair r, block of step k).  The cells are added up
  // after the walk, when the walk's registers are free.
  unsigned long long mine = 0;
  auto settle = [&](int k, int oldv) {
#pragma unroll
    for (int r = 0; r < RB; ++r)
      if (__builtin_amdgcn_readlane(oldv, r) == NU - 1) mine |= 1ull << (RB * k + r);
  };
  int old[DEPTH] = {0, 0};
  for (int k0 = 0; k0 < n; k0 += DEPTH) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      const int k = k0 + d;
      if (k < n) {
        float t[RB][G1];
        down_terms<GS, RB>(st[d], sc, t);
        // step k's weights are here, so everything this wave issued before requesting them is complete: the terms of
        // step k - 2 are acknowledged and its count may go; the count issued at step k - 2 (for step k - 4) is back
        asm volatile("" : "+v"(t[0][0]) : : "memory");
        if (k >= 2 * DEPTH) settle(k - 2 * DEPTH, old[d]);
        if (k >= DEPTH) old[d] = bump(k - DEPTH);
        const int db = walk.db(k);
        if (walk.col_ok(k)) {
#pragma unroll
          for (int r = 0; r < RB; ++r)
#pragma unroll
            for (int gi = 0; gi < G1; ++gi)
              if (gi < walk.ng)
                st_agent(sa.part + (((size_t)pr[r] * NBD2 + db) * KG + walk.g0 + gi) * 64 + lane, t[r][gi]);
        }
        __atomic_signal_fence(__ATOMIC_SEQ_CST);        // the refill below stays behind these stores
        if (k + DEPTH < n) walk.load(st[d], k + DEPTH);
      }
    }
  }
  __builtin_amdgcn_s_waitcnt(0);
  // what is still open: the counts issued at the last two steps, and the last two steps' own
  for (int k = max(n - DEPTH, DEPTH); k < n; ++k) settle(k - DEPTH, (k & 1) ? old[1] : old[0]);
  for (int k = max(n - DEPTH, 0); k < n; ++k) settle(k, bump(k));

  // The cells this wave completed.  (pair p, block db) has all its groups: the pair's output; and if that completes
  // the token's cell too, the token's.
  while (mine) {
    const int bit = __builtin_ctzll(mine);
    mine &= mine - 1;
    const int p = (RB == 2 && (bit & 1)) ? pr[RB - 1] : pr[0], db = walk.db(bit / RB);
    const int col = db * 64 + lane;
    const size_t cell = (size_t)p * NBD2 + db;
    if (lane == 0) __hip_atomic_store(sa.c1 + cell * TF_ARRIVE_STRIDE, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const float yv = slice_tree(sa.part + cell * KG * 64 + lane, KG);
    if (col < D) st_agent(sa.y + (size_t)p * D + col, yv);
    __builtin_amdgcn_s_waitcnt(0);                    // the pair's output is acknowledged, then it counts
    const int token = p / slots;
    int done = 0;
    if (lane == 0) {
      int* c = sa.c2 + ((size_t)token * NBD2 + db) * TF_ARRIVE_STRIDE;
      done = __hip_atomic_fetch_add(c, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == slots - 1;
      if (done) __hip_atomic_store(c, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    if (!__builtin_amdgcn_readfirstlane(done)) continue;
    // the token's weights: lane k holds slot k's
    float w = 0.f;
    if (L) {
      int id;
      topk_lane(L + (size_t)token * ldl, NE, TOPK, shared, lane, id, w);
    } else if (lane < slots) {
      w = sa.wts[(size_t)token * slots + lane];
    }
    float a = 0.f;
    for (int k0 = 0; k0 < slots; k0 += 8) {
      float v[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int k = k0 + j < slots ? k0 + j : slots - 1;
        v[j] = col < D ? ld_agent(sa.y + ((size_t)token * slots + k) * D + col) : 0.f;
      }
#pragma unroll
      for (int j = 0; j < 8; ++j)
        if (k0 + j < slots) a = fmaf(__shfl(w, k0 + j), v[j], a);
    }
    if (col < D) sa.out[(size_t)token * D + col] = (uint16_t)f32_bf16_bits(a);
  }
}

// Up unit, then its part of the down projection (see above).  Every thread of the workgroup calls this.
template <int GS, int NM, int EPI, int WAVES>
__device__ __forceinline__ void sliced_unit(const uint16_t* __restrict__ X, int64_t x_stride, int slots,
                                            const uint32_t* __restrict__ Wup, int D, int NI, int e, int cnt,
                                            const int* pairs, int cb2, uint16_t* __restrict__ act, float limit, float* lds,
                                            const SliceArgs& sa, const float* __restrict__ L, int64_t ldl, int NE,
                                            int TOPK, int shared) {
  __shared__ uint32_t actw[RBMAX * 32];
  const int tid = threadIdx.x;
  DownWalk<GS, WAVES> walk;
  walk.NBd = D / 32;
  walk.NBD2 = (walk.NBd + 1) >> 1;
  walk.KGd = NI / GS;
  walk.g0 = cb2 * (64 / GS);
  walk.ng = min(64 / GS, walk.KGd - walk.g0);
  const int NU = (NI / 32 + 1) >> 1;
  walk.rot = (int)((long long)cb2 * walk.NBD2 / NU);
  walk.wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  walk.lane = tid & 63;
  walk.n = walk.wave < walk.NBD2 ? (walk.NBD2 - walk.wave + WAVES - 1) / WAVES : 0;
  walk.wexp = sa.Wdown + (size_t)e * walk.NBd * walk.KGd * block_words(GS);
  DownStage<GS> st[DEPTH];
  struct Sink {
    const DownWalk<GS, WAVES>& walk;
    DownStage<GS> (&st)[DEPTH];
    uint32_t* actw;
    // the first steps of the down walk are requested before the up projection's sums meet
    __device__ __forceinline__ void streamed() const {
#pragma unroll
      for (int d = 0; d < DEPTH; ++d)
        if (d < walk.n) walk.load(st[d], d);
    }
    __device__ __forceinline__ void act(int r, int l, uint32_t bits) const {
      reinterpret_cast<uint16_t*>(actw)[r * 64 + l] = (uint16_t)bits;
    }
  } sink{walk, st, actw};
  NoHook none;
  expert_unit<GS, NM, EPI, WAVES, 0>(X, x_stride, slots, Wup, D / GS, NI / 32, e, cnt, pairs, cb2, act, NI, limit, lds, none,
                                     sink);
  __syncthreads();          // the rows' activations are in LDS
  if (cnt == 2) down_slices<GS, WAVES, 2>(walk, st, pairs, actw, slots, D, NU, sa, L, ldl, NE, TOPK, shared);
  else down_slices<GS, WAVES, 1>(walk, st, pairs, actw, slots, D, NU, sa, L, ldl, NE, TOPK, shared);
}

// ---- routing and the up projection in one launch -------------------------------------------------------------------
//
// Workgroup 0 writes the routing's outputs (picks, weights, members, items, counts, item descriptors) for the kernels
// that follow; every other workgroup repeats the cheap part for itself (top-k of every row, a histogram, one scan)
// to learn which expert and which pairs its item holds, then runs the up unit.  The routing's launch and its trip
// through memory are gone; the price is about a microsecond of arithmetic at the head of each workgroup.

template <int GS, int NM, int EPI, int WAVES, bool SLICED = false>
__global__ void __launch_bounds__(WAVES * 64)
    route_up_kernel(const float* __restrict__ L, int64_t ldl, int R, int NE, int TOPK, int shared,
                    const uint16_t* __restrict__ X, int64_t x_stride, const uint32_t* __restrict__ Wup, int D, int NI,
                    int* __restrict__ pick, float* __restrict__ wts, int* __restrict__ members,
                    int* __restrict__ items, int* __restrict__ counts, int* __restrict__ desc,
                    uint16_t* __restrict__ act, float limit, int* __restrict__ zero, int n_zero, SliceArgs sa) {
  extern __shared__ float lds[];
  __shared__ int pk[PLAN_THREADS];
  __shared__ ItemLds item;
  TF_MARK(0);
  __builtin_amdgcn_s_setprio(3);       // the lookup issues ahead of the workgroups that already stream
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, threads = WAVES * 64;
  const int slots = TOPK + (shared ? 1 : 0), P = R * slots, E = NE + (shared ? 1 : 0);
  const bool writer = blockIdx.x == 0;
  // the workgroup's unit: the up projection alone, or (SLICED) with its part of the down projection behind it
  auto unit = [&](int e, int cnt, const int* pairs, int cb2) {
    if constexpr (SLICED) {
      sliced_unit<GS, NM, EPI, WAVES>(X, x_stride, slots, Wup, D, NI, e, cnt, pairs, cb2, act, limit, lds, sa, L, ldl, NE,
                                      TOPK, shared);
    } else {
      NoHook none;
      expert_unit<GS, NM, EPI, WAVES, 0>(X, x_stride, slots, Wup, D / GS, NI / 32, e, cnt, pairs, cb2, act, NI, limit, lds,
                                         none);
    }
  };
  auto keep = [&](int r, int id, float w) {
    if (lane < slots) {
      pk[r * slots + lane] = (unsigned)id < (unsigned)E ? id : -1;
      if (writer) {
        pick[r * slots + lane] = id;
        wts[r * slots + lane] = w;
      }
    }
  };
  const int NB2 = (NI / 32 + 1) >> 1;
  const int u = blockIdx.x - 1, it = u / NB2, cb2 = u - it * NB2;
  if (R == 1 && !writer) {
    // one row: every pick is its own item, so unit `it` takes slot `it`, and needs the selection only up to it
    if (it >= slots) return;
    if (wave == 0) {
      int id;
      if (!L) {
        id = pick[it];
      } else if (shared && it == TOPK) {
        id = NE;
      } else if (NE <= 128) {
        float v[2];
        topk_load<2>(L, NE, lane, v);
        id = topk_kth<2>(v, it, lane);
      } else if (NE <= 512) {
        float v[8];
        topk_load<8>(L, NE, lane, v);
        id = topk_kth<8>(v, it, lane);
      } else {
        float v[TOPK_VPL];
        topk_load<TOPK_VPL>(L, NE, lane, v);
        id = topk_kth<TOPK_VPL>(v, it, lane);
      }
      if (lane == 0) {
        item.sel[0] = (unsigned)id < (unsigned)E ? id : -1;
        item.sel[2] = 1;
        item.pairs[0] = it;
      }
    }
    __syncthreads();
    if (item.sel[0] < 0) return;
    unit(item.sel[0], 1, item.pairs, cb2);
    return;
  }
  if (L && !writer && R <= 64) {
    // a workgroup a pair (and 64 columns): the item is found from the pair's own row and one look at the others
    __shared__ int wavepairs[WAVES][2];
    if (it >= P) return;
    int e = 0, cnt = 0;
    const bool live =
        NE <= 128 ? pair_item<2, WAVES>(L, ldl, R, NE, TOPK, shared, slots, it, pk, item.sel, wavepairs[wave], e, cnt)
        : NE <= 512 ? pair_item<8, WAVES>(L, ldl, R, NE, TOPK, shared, slots, it, pk, item.sel, wavepairs[wave], e, cnt)
                    : pair_item<TOPK_VPL, WAVES>(L, ldl, R, NE, TOPK, shared, slots, it, pk, item.sel, wavepairs[wave], e, cnt);
    if (!live) return;
    unit(e, cnt, wavepairs[wave], cb2);
    return;
  }
  if (!L && !writer) {
    // the picks are given: a workgroup a pair, its item from the picks alone
    __shared__ int wavepairs[WAVES][2];
    if (it >= P) return;
    int e = 0, cnt = 0;
    if (!pair_item_given(pick, P, E, it, wavepairs[wave], e, cnt)) return;
    unit(e, cnt, wavepairs[wave], cb2);
    return;
  }
  for (int e = tid; e < E; e += threads) item.cnt[e] = 0;
  if (tid < 6) item.sel[tid] = tid == 0 ? -1 : 0;
  __syncthreads();
  auto count = [&](int id) {
    if ((unsigned)id >= (unsigned)E || writer) return;
    const int old = atomicAdd(&item.cnt[id], 1);
    if (old % DTILE == DTILE - 1) atomicAdd(&item.sel[5], 1);
  };
  if (!L) {
    // the picks are given (a top-k launch ran before): only the plan is made here
    for (int p = tid; p < P; p += threads) {
      pk[p] = (unsigned)pick[p] < (unsigned)E ? pick[p] : -1;
      count(pk[p]);
    }
  } else if (NE <= 128 && slots <= 16 && R > WAVES) {
    // more rows than waves: four logits rows a wave, each on a row of 16 lanes
    for (int r0 = 4 * wave; r0 < R; r0 += 4 * WAVES) {
      const int r = r0 + (lane >> 4);
      int id;
      float w;
      topk_row16(r < R ? L + (size_t)r * ldl : nullptr, NE, TOPK, shared, lane, id, w);
      if (r < R && (lane & 15) < slots) {
        pk[r * slots + (lane & 15)] = (unsigned)id < (unsigned)E ? id : -1;
        count(id);
        if (writer) {
          pick[r * slots + (lane & 15)] = id;
          wts[r * slots + (lane & 15)] = w;
        }
      }
    }
  } else {
    for (int r = wave; r < R; r += WAVES) {
      int id;
      float w;
      topk_lane(L + (size_t)r * ldl, NE, TOPK, shared, lane, id, w);
      keep(r, id, w);
      if (lane < slots) count(id);
    }
  }
  __syncthreads();
  if (writer) {
    for (int i = tid; i < n_zero; i += threads) zero[i] = 0;      // the next launch's arrival counters
    // the whole plan: first member and first item of every expert (wave 0 scans), then items, members, descriptors
    int* off = reinterpret_cast<int*>(lds);
    int* itoff = off + EMAX;
    int* dtoff = itoff + EMAX;                 // descriptors: an expert's first full item; full items come first
    int* shoff = dtoff + EMAX;                 // and its short last item among the short ones, which follow
    for (int e = tid; e < E; e += threads) item.cnt[e] = 0;
    __syncthreads();
    for (int p = tid; p < P; p += threads)
      if (pk[p] >= 0) atomicAdd(&item.cnt[pk[p]], 1);
    __syncthreads();
    if (tid < 64) {
      int items_before = 0, pairs_before = 0, full_before = 0, short_before = 0, used = 0;
      for (int e0 = 0; e0 < E; e0 += 64) {
        const int e = e0 + lane, c = e < E ? item.cnt[e] : 0, t = (c + 15) >> 4, f = c / DTILE,
                  r = c - DTILE * f > 0 ? 1 : 0;
        const int ti = wave_scan(t), ci = wave_scan(c), fi = wave_scan(f), ri = wave_scan(r);
        if (e < E) {
          off[e] = pairs_before + ci - c;
          itoff[e] = items_before + ti - t;
          dtoff[e] = full_before + fi - f;
          shoff[e] = short_before + ri - r;
        }
        items_before += __builtin_amdgcn_readlane(ti, 63);
        pairs_before += __builtin_amdgcn_readlane(ci, 63);
        full_before += __builtin_amdgcn_readlane(fi, 63);
        short_before += __builtin_amdgcn_readlane(ri, 63);
        used += __popcll(__ballot(c > 0));
      }
      if (lane == 0) {
        counts[0] = items_before;
        counts[1] = used;
        desc[0] = full_before + short_before;
        item.sel[5] = full_before;
      }
    }
    __syncthreads();
    const int F = item.sel[5];
    for (int e = tid; e < E; e += threads) {
      const int c = item.cnt[e];
      for (int j = 0; 16 * j < c; ++j) {
        const int i = itoff[e] + j, first = off[e] + 16 * j, n = min(16, c - 16 * j);
        items[3 * i] = e;
        items[3 * i + 1] = first;
        items[3 * i + 2] = n;
      }
      for (int j = 0; DTILE * j < c; ++j) {
        const int n = min(DTILE, c - DTILE * j);
        int* d = desc + (size_t)(1 + (n == DTILE ? dtoff[e] + j : F + shoff[e])) * DESC;
        d[0] = e;
        d[1] = n;
        d[2] = off[e] + DTILE * j;
        d[3] = 0;
      }
    }
    // a wave an expert that has pairs: its members in pair order, and their places in its descriptors
    for (int e = wave; e < E; e += WAVES) {
      const int c = item.cnt[e];
      if (!c) continue;
      expert_pairs(pk, P, e, c, lane, [&](int rank, int p) {
        members[off[e] + rank] = p;
        const int j = rank / DTILE, row = DTILE * (j + 1) <= c ? dtoff[e] + j : F + shoff[e];
        desc[(size_t)(1 + row) * DESC + 4 + rank % DTILE] = p;
      });
    }
    return;
  }
  if (!find_item<DTILE, true>(item, pk, P, E, it)) return;
  // the item's rows are summed group by group inside the unit (a pass at a time), under its first weight loads
  unit(item.sel[0], item.sel[2], item.pairs, cb2);
}

template <int GS, int NM, int EPI, bool SLICED = false>
int launch_route_up(const float* logits, int64_t ldl, int rows, int experts, int top_k, int shared, const uint16_t* x,
                    int64_t x_stride, const uint32_t* wup, int d, int ni, int* pick, float* wts, int* members,
                    int* items, int* counts, int* desc, uint16_t* act, float limit, int max_items, int* zero,
                    int n_zero, hipStream_t stream, const SliceArgs& sa = SliceArgs{}) {
  const int nb2 = (ni / 32 + 1) / 2;
  // with the picks given, or logits of 2 to 64 rows, the workgroups go a pair (route_up_kernel), else an item
  const int64_t pairs = (int64_t)rows * (top_k + (shared ? 1 : 0));
  const int64_t units = !logits || (rows > 1 && rows <= 64) ? pairs : max_items;
  const int64_t grid = 1 + units * nb2;
  TF_REQUIRE(grid <= 0x7FFFFFFF, "moe: %lld workgroups exceed the grid limit", (long long)grid);
  const size_t floats = expert_lds_floats(NM);
  const size_t smem = sizeof(float) * (floats > 4 * EMAX ? floats : 4 * EMAX);
  TF_REQUIRE(smem <= 48 * 1024, "moe: %d input groups need %zu bytes of LDS", d / GS, smem);
  const dim3 g((unsigned)grid);
#define TF_GO(W_)                                                                                              \
  route_up_kernel<GS, NM, EPI, W_, SLICED><<<g, W_ * 64, smem, stream>>>(logits, ldl, rows, experts, top_k, shared, x, \
                                                                         x_stride, wup, d, ni, pick, wts, members,    \
                                                                         items, counts, desc, act, limit, zero,       \
                                                                         n_zero, sa)
  switch (SLICED ? sliced_waves(grid) : fused_waves(2 * grid)) {
    case 16: TF_GO(16); break;
    case 8: TF_GO(8); break;
    default: TF_GO(4);
  }
#undef TF_GO
  TF_LAUNCH_OK(SLICED ? "tf_moe_decode_sliced" : "tf_moe_route_up");
  return 0;
}

template <int GS, int NM, int EPI_UP>
int launch_fused(const uint16_t* x, int64_t x_stride, int slots, const uint32_t* wup, const uint32_t* wdown, int d,
                 int ni, const int* desc, const int* counts, const float* wts, uint16_t* act, float* y, uint16_t* out, int* done, int* arrive, int* status, float limit,
                 int max_items, int astride, hipStream_t stream) {
  const int nb2u = (ni / 32 + 1) / 2, nb2d = (d / 32 + 1) / 2;
  const int64_t grid = (int64_t)max_items * (nb2u + nb2d);
  if (grid < 1) return 0;
  TF_REQUIRE(grid <= 0x7FFFFFFF, "moe: %lld workgroups exceed the grid limit", (long long)grid);
  const size_t smem = sizeof(float) * expert_lds_floats(NM);
  const int spins = 1 << 16;     // polls of about a microsecond: far past any real wait, short enough to drain fast
  const dim3 g((unsigned)grid);
#define TF_GO(W_)                                                                                                 \
  moe_fused_kernel<GS, NM, EPI_UP, W_><<<g, W_ * 64, smem, stream>>>(x, x_stride, slots, wup, wdown, d, ni, desc, \
                                                                     counts, wts, act, y, out, done,              \
                                                                     arrive, status, limit, max_items, spins, astride)
  switch (fused_waves(grid)) {
    case 16: TF_GO(16); break;
    case 8: TF_GO(8); break;
    default: TF_GO(4);
  }
#undef TF_GO
  TF_LAUNCH_OK("tf_moe_decode_experts");
  return 0;
}

}  // namespace
}  // namespace tf

using namespace tf;

TF_TIMELINE_EXPORT(moe)

extern "C" int tf_moe_decode_experts(int gs, int swiglu, const uint16_t* x, int64_t x_stride, int rows, int slots,
                                     const uint32_t* up, const uint32_t* down, int d, int ni, const int32_t* desc,
                                     const int32_t* counts, const float* wts, uint16_t* act, float* y,
                                     uint16_t* out, int32_t* done, int32_t* arrive,
                                     int32_t* status, float limit, int max_items, tf_stream_t stream) {
  clear_error();
  TF_REQUIRE(gs == 32 || gs == 64, "moe: groups of 32 or 64 inputs, not %d", gs);
  TF_REQUIRE(x && up && down && desc && counts && wts && act && y && out && done && arrive && status,
             "moe: null pointer argument");
  TF_REQUIRE(d % 64 == 0 && ni % 64 == 0 && d % gs == 0 && ni % gs == 0,
             "moe: the fused decode layer takes hidden and intermediate sizes that are multiples of 64");
  TF_REQUIRE(aligned16(x) && x_stride % 8 == 0 && aligned16(up) && aligned16(down) && aligned16(act),
             "x: rows of K = groups * group size inputs, 16-byte aligned");
  TF_REQUIRE(rows >= 1 && slots >= 1 && max_items >= 1, "moe: empty call");
  hipStream_t s = as_stream(stream);
  if (gs == 64)
    return swiglu ? launch_fused<64, 2, 2>(x, x_stride, slots, up, down, d, ni, desc, counts, wts, act, y,
                                           out, done, arrive, status, limit, max_items, arrive_stride(rows), s)
                  : launch_fused<64, 1, 1>(x, x_stride, slots, up, down, d, ni, desc, counts, wts, act, y,
                                           out, done, arrive, status, limit, max_items, arrive_stride(rows), s);
  return swiglu ? launch_fused<32, 2, 2>(x, x_stride, slots, up, down, d, ni, desc, counts, wts, act, y,
                                         out, done, arrive, status, limit, max_items, arrive_stride(rows), s)
                : launch_fused<32, 1, 1>(x, x_stride, slots, up, down, d, ni, desc, counts, wts, act, y,
                                         out, done, arrive, status, limit, max_items, arrive_stride(rows), s);
}

extern "C" int tf_moe_route_up(const float* logits, int64_t ldl, int rows, int experts, int top_k, int shared, int gs,
                               int swiglu, const uint16_t* x, int64_t x_stride, const uint32_t* up, int d, int ni,
                               int32_t* pick, float* wts, int32_t* members, int32_t* items, int32_t* counts,
                               int32_t* desc, uint16_t* act, float limit, int max_items, int32_t* zero, int n_zero,
                               tf_stream_t stream) {
  clear_error();
  TF_REQUIRE(gs == 32 || gs == 64, "moe: groups of 32 or 64 inputs, not %d", gs);
  TF_REQUIRE(x && up && pick && wts && members && items && counts && desc && act, "moe: null pointer argument");
  TF_REQUIRE(experts >= 1 && experts + (shared ? 1 : 0) <= EMAX && experts <= 64 * TOPK_VPL,
             "route: at most %d experts", EMAX - 1);
  TF_REQUIRE(top_k >= 1 && top_k + (shared ? 1 : 0) <= 64 && top_k <= experts, "route: 1 to 64 slots a row, not %d",
             top_k);
  TF_REQUIRE(rows >= 1 && (int64_t)rows * (top_k + (shared ? 1 : 0)) <= PLAN_THREADS,
             "route: the decode routing takes at most %d pairs", PLAN_THREADS);
  TF_REQUIRE(!logits || ldl >= experts + (shared ? 1 : 0), "route: logits rows are too short");
  TF_REQUIRE(d % gs == 0 && ni % 32 == 0 && ni % gs == 0 && d >= gs && max_items >= 1,
             "moe: hidden and intermediate sizes in whole groups and 32-column blocks");
  TF_REQUIRE(aligned16(x) && x_stride % 8 == 0 && aligned16(up) && aligned16(act),
             "x: rows of K = groups * group size inputs, 16-byte aligned");
  TF_REQUIRE(n_zero >= 0 && (n_zero == 0 || zero), "route: bad counter range");
  hipStream_t s = as_stream(stream);
  if (gs == 64)
    return swiglu ? launch_route_up<64, 2, 2>(logits, ldl, rows, experts, top_k, shared, x, x_stride, up, d, ni, pick,
                                              wts, members, items, counts, desc, act, limit, max_items, zero, n_zero, s)
                  : launch_route_up<64, 1, 1>(logits, ldl, rows, experts, top_k, shared, x, x_stride, up, d, ni, pick,
                                              wts, members, items, counts, desc, act, limit, max_items, zero, n_zero, s);
  return swiglu ? launch_route_up<32, 2, 2>(logits, ldl, rows, experts, top_k, shared, x, x_stride, up, d, ni, pick, wts,
                                            members, items, counts, desc, act, limit, max_items, zero, n_zero, s)
                : launch_route_up<32, 1, 1>(logits, ldl, rows, experts, top_k, shared, x, x_stride, up, d, ni, pick, wts,
                                            members, items, counts, desc, act, limit, max_items, zero, n_zero, s);
}

extern "C" int tf_moe_decode_sliced(const float* logits, int64_t ldl, int rows, int experts, int top_k, int shared, int gs,
                                    int swiglu, const uint16_t* x, int64_t x_stride, const uint32_t* up,
                                    const uint32_t* down, int d, int ni, int32_t* pick, float* wts, int32_t* members,
                                    int32_t* items, int32_t* counts, int32_t* desc, uint16_t* act, float* y,
                                    uint16_t* out, float* part, int32_t* arrive, float limit, int max_items,
                                    tf_stream_t stream) {
  clear_error();
  TF_REQUIRE(gs == 32 || gs == 64, "moe: groups of 32 or 64 inputs, not %d", gs);
  TF_REQUIRE(x && up && down && pick && wts && members && items && counts && desc && act && y && out && part && arrive,
             "moe: null pointer argument");
  TF_REQUIRE(experts >= 1 && experts + (shared ? 1 : 0) <= EMAX && experts <= 64 * TOPK_VPL,
             "route: at most %d experts", EMAX - 1);
  TF_REQUIRE(top_k >= 1 && top_k + (shared ? 1 : 0) <= 64 && top_k <= experts, "route: 1 to 64 slots a row, not %d",
             top_k);
  TF_REQUIRE(rows >= 1 && (int64_t)rows * (top_k + (shared ? 1 : 0)) <= PLAN_THREADS,
             "route: the decode routing takes at most %d pairs", PLAN_THREADS);
  TF_REQUIRE(!logits || ldl >= experts + (shared ? 1 : 0), "route: logits rows are too short");
  TF_REQUIRE(d % 64 == 0 && ni % 64 == 0 && d % gs == 0 && ni % gs == 0 && d >= gs && max_items >= 1,
             "moe: the sliced decode layer takes hidden and intermediate sizes that are multiples of 64");
  TF_REQUIRE(d <= 8192, "moe: the sliced decode layer takes a hidden size of at most 8192, not %d", d);
  TF_REQUIRE(aligned16(x) && x_stride % 8 == 0 && aligned16(up) && aligned16(down) && aligned16(act),
             "x: rows of K = groups * group size inputs, 16-byte aligned");
  hipStream_t s = as_stream(stream);
  const int pairs = rows * (top_k + (shared ? 1 : 0));
  SliceArgs sa;
  sa.Wdown = down;
  sa.part = part;
  sa.y = y;
  sa.out = out;
  sa.c1 = arrive;
  sa.c2 = arrive + (size_t)pairs * (d / 64) * TF_ARRIVE_STRIDE;
  sa.wts = wts;
#define TF_SL(GS_, NM_, EPI_)                                                                                          \
  launch_route_up<GS_, NM_, EPI_, true>(logits, ldl, rows, experts, top_k, shared, x, x_stride, up, d, ni, pick, wts, \
                                        members, items, counts, desc, act, limit, max_items, nullptr, 0, s, sa)
  if (gs == 64) return swiglu ? TF_SL(64, 2, 2) : TF_SL(64, 1, 1);
  return swiglu ? TF_SL(32, 2, 2) : TF_SL(32, 1, 1);
#undef TF_SL
}

extern "C" int tf_moe_down_combine(int gs, const uint16_t* act, int rows, int slots, const uint32_t* down, int d, int ni,
                                   const int32_t* desc, const float* wts, float* y, uint16_t* out, int32_t* arrive,
                                   int max_items, tf_stream_t stream) {
  clear_error();
  TF_REQUIRE(gs == 32 || gs == 64, "moe: groups of 32 or 64 inputs, not %d", gs);
  TF_REQUIRE(act && down && desc && wts && y && out && arrive, "moe: null pointer argument");
  TF_REQUIRE(d % 32 == 0 && ni % gs == 0 && ni >= gs && rows >= 1 && slots >= 1 && max_items >= 1,
             "moe: hidden size in 32-column blocks, intermediate size in whole groups");
  TF_REQUIRE(aligned16(act) && ni % 8 == 0 && aligned16(down), "act: rows of whole groups, 16-byte aligned");
  const int nb2 = (d / 32 + 1) / 2;
  const int64_t grid = (int64_t)max_items * nb2;
  TF_REQUIRE(grid <= 0x7FFFFFFF, "moe: %lld workgroups exceed the grid limit", (long long)grid);
  const size_t smem = sizeof(float) * expert_lds_floats(1);
  hipStream_t s = as_stream(stream);
  const dim3 g((unsigned)grid);
#define TF_GO(GS_, W_)                                                                                             \
  down_combine_kernel<GS_, W_><<<g, W_ * 64, smem, s>>>(act, slots, down, d, ni, desc, wts, y, out, arrive, \
                                                        arrive_stride(rows))
#define TF_GS(GS_)                      \
  switch (fused_waves(grid)) {                 \
    case 16: TF_GO(GS_, 16); break;     \
    case 8: TF_GO(GS_, 8); break;       \
    default: TF_GO(GS_, 4);             \
  }
  if (gs == 64) { TF_GS(64) } else { TF_GS(32) }
#undef TF_GS
#undef TF_GO
  TF_LAUNCH_OK("tf_moe_down_combine");
  return 0;
}
