// Routing pieces shared by the routing kernels and the decode kernels that route for themselves: the per-row top-k
// (one wave a row), block-wide scans, and the lookup of one item of the pair sort without building the whole plan.
#pragma once

#include "tf_common.h"

namespace tf {
namespace {

// ---- top-k: one wave a row ------------------------------------------------------------------------------------------

constexpr int TOPK_VPL = 16;     // values a lane: up to 1024 experts

// Maximum over the 64 lanes, the same value in every lane: a butterfly inside each row of 16 lanes through DPP
// (no LDS round trips), then the four rows' maxima through readlane.
__device__ __forceinline__ float wave_max(float x) {
#define TF_DPP(V_, CTRL_) \
  __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, V_), CTRL_, 0xf, 0xf, false))
  x = fmaxf(x, TF_DPP(x, 0xB1));        // quad_perm [1, 0, 3, 2]
  x = fmaxf(x, TF_DPP(x, 0x4E));        // quad_perm [2, 3, 0, 1]
  x = fmaxf(x, TF_DPP(x, 0x141));       // row_half_mirror
  x = fmaxf(x, TF_DPP(x, 0x140));       // row_mirror
#undef TF_DPP
  auto row = [&](int l) { return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, x), l)); };
  return fmaxf(fmaxf(row(0), row(16)), fmaxf(row(32), row(48)));
}

// one wave, one row (see tf_moe_topk): lane k < TOPK leaves with the k-th pick and its weight, lane TOPK with the
// shared expert's when there is one.  VPL values a lane cover 64 * VPL experts.
template <int VPL>
__device__ __forceinline__ void topk_load(const float* __restrict__ row, int NE, int lane, float (&v)[VPL]) {
#pragma unroll
  for (int i = 0; i < VPL; ++i) {
    const int e = lane + 64 * i;
    v[i] = e < NE ? row[e] : -__builtin_inff();
  }
}

template <int VPL>
__device__ __forceinline__ void topk_pick(float (&v)[VPL], const float* __restrict__ row, int NE, int TOPK, int shared,
                                          int lane, int& id, float& w) {
  const float NEG = -__builtin_inff();
  float mine_m = 0.f;
  int mine_id = 0;
  for (int k = 0; k < TOPK; ++k) {
    float bv = v[0];
    int bi = lane;
#pragma unroll
    for (int i = 1; i < VPL; ++i)
      if (v[i] > bv) {
        bv = v[i];
        bi = lane + 64 * i;
      }
    const float m = wave_max(bv);
    // the lowest expert id among the lanes that hold the maximum (nearly always one lane)
    unsigned long long cand = __ballot(bv == m);
    int idx = 0x7FFFFFFF;
    while (cand) {
      const int l = __builtin_ctzll(cand);
      idx = min(idx, __builtin_amdgcn_readlane(bi, l));
      cand &= cand - 1;
    }
    if (lane == k) {
      mine_m = m;
      mine_id = idx;
    }
    if ((idx & 63) == lane) {
#pragma unroll
      for (int i = 0; i < VPL; ++i)
        if (i == (idx >> 6)) v[i] = NEG;
    }
  }
  // weights: exp(l_k - l_0) over their sum, added in pick order (lane k holds pick k)
  const float top = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, mine_m), 0));
  const float ex = expf(mine_m - top);
  float total = 0.f;
  for (int k = 0; k < TOPK; ++k)
    total += __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, ex), k));
  id = mine_id;
  w = round_bf16(ex / total);
  if (shared && lane == TOPK) {
    const float sg = round_bf16(row[NE]);
    id = NE;
    w = round_bf16(1.f / (1.f + expf(-sg)));
  }
}

// Up to 128 experts and 16 slots: a logits row on a ROW of 16 lanes (eight values a lane), four logits rows a wave.
// Every reduction stays inside the 16 lanes (DPP), so the four rows cost one row's instructions.  `row` is this
// lane group's logits row, or null when it has none.  Lane k of the group (k < TOPK) leaves with pick k and its
// weight, lane TOPK with the shared expert's.  The arithmetic, and so every bit, is topk_pick's.
__device__ __forceinline__ void topk_row16(const float* __restrict__ row, int NE, int TOPK, int shared, int lane,
                                           int& id, float& w) {
#define TF_ROW_F(V_, CTRL_) \
  __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, V_), CTRL_, 0xf, 0xf, false))
#define TF_ROW_I(V_, CTRL_) __builtin_amdgcn_update_dpp(0, V_, CTRL_, 0xf, 0xf, false)
  const float NEG = -__builtin_inff();
  const int l = lane & 15;
  float v[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int e = l + 16 * i;
    v[i] = row && e < NE ? row[e] : NEG;
  }
  float mine_m = 0.f;
  int mine_id = 0;
  for (int k = 0; k < TOPK; ++k) {
    float bv = v[0];
    int bi = l;
#pragma unroll
    for (int i = 1; i < 8; ++i)
      if (v[i] > bv) {
        bv = v[i];
        bi = l + 16 * i;
      }
    float m = bv;
    m = fmaxf(m, TF_ROW_F(m, 0xB1));         // quad_perm [1, 0, 3, 2]
    m = fmaxf(m, TF_ROW_F(m, 0x4E));         // quad_perm [2, 3, 0, 1]
    m = fmaxf(m, TF_ROW_F(m, 0x141));        // row_half_mirror
    m = fmaxf(m, TF_ROW_F(m, 0x140));        // row_mirror
    int idx = bv == m ? bi : 0x7FFFFFFF;     // the lowest id among the lanes that hold the maximum
    idx = min(idx, TF_ROW_I(idx, 0xB1));
    idx = min(idx, TF_ROW_I(idx, 0x4E));
    idx = min(idx, TF_ROW_I(idx, 0x141));
    idx = min(idx, TF_ROW_I(idx, 0x140));
    if (l == k) {
      mine_m = m;
      mine_id = idx;
    }
    if ((idx & 15) == l) {
#pragma unroll
      for (int i = 0; i < 8; ++i)
        if (i == (idx >> 4)) v[i] = NEG;
    }
  }
  const float top = TF_ROW_F(mine_m, 0x150);                // row_newbcast:0
  const float ex = l < TOPK ? expf(mine_m - top) : 0.f;
  float sum = ex;                                           // lane j ends with ((e0 + e1) + ...) + ej
  for (int k = 1; k < TOPK; ++k) sum = TF_ROW_F(sum, 0x111) + ex;     // row_shr:1, zero shifted in
  const float total = __shfl(sum, (lane & 48) + TOPK - 1);
  id = mine_id;
  w = round_bf16(ex / total);
  if (shared && l == TOPK && row) {
    const float sg = round_bf16(row[NE]);
    id = NE;
    w = round_bf16(1.f / (1.f + expf(-sg)));
  }
#undef TF_ROW_F
#undef TF_ROW_I
}

// The k-th pick of a row alone: passes 0 .. k of topk_pick's selection (value descending, ties to the lower id), no
// weights.  The same value in every lane.
template <int VPL>
__device__ __forceinline__ int topk_kth(float (&v)[VPL], int k, int lane) {
  const float NEG = -__builtin_inff();
  int idx = 0;
  for (int pass = 0; pass <= k; ++pass) {
    float bv = v[0];
    int bi = lane;
#pragma unroll
    for (int i = 1; i < VPL; ++i)
      if (v[i] > bv) {
        bv = v[i];
        bi = lane + 64 * i;
      }
    const float m = wave_max(bv);
    unsigned long long cand = __ballot(bv == m);
    idx = 0x7FFFFFFF;
    while (cand) {
      const int l = __builtin_ctzll(cand);
      idx = min(idx, __builtin_amdgcn_readlane(bi, l));
      cand &= cand - 1;
    }
    if ((idx & 63) == lane) {
#pragma unroll
      for (int i = 0; i < VPL; ++i)
        if (i == (idx >> 6)) v[i] = NEG;
    }
  }
  return idx;
}

// The slot expert e would take in a row (v as topk_load leaves it): the number of experts that the selection takes
// before it, i.e. with a larger logit, or an equal one and a lower id.  e is picked iff this is below TOPK, and
// then it is the pick's slot, since the passes of topk_pick take the experts in exactly that order.
template <int VPL>
__device__ __forceinline__ int topk_slot_of(const float (&v)[VPL], int e, int lane) {
  float c = v[0];
#pragma unroll
  for (int i = 1; i < VPL; ++i)
    if (i == (e >> 6)) c = v[i];
  const float val = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, c), e & 63));
  int rank = 0;
#pragma unroll
  for (int i = 0; i < VPL; ++i) rank += __popcll(__ballot(v[i] > val || (v[i] == val && lane + 64 * i < e)));
  return rank;
}

// A workgroup that takes ONE pair p = (row r, slot k) finds its item without the other rows' top-k: wave 0 runs
// k + 1 selection passes over row r to learn the expert; every wave then asks of its share of the rows whether the
// expert is among their picks (topk_slot_of); the expert's pairs, in pair order, go two an item, and the workgroup
// of an item's first pair takes the item, the workgroup of its second pair leaves.  Items and their pairs are those
// of the plan's descriptors (DTILE = 2).  R <= 64.  memb: R ints of LDS, sel: one, wp: this wave's two.
// Every thread calls this (two barriers).  False: this workgroup has nothing to do.
template <int VPL, int WAVES>
__device__ __forceinline__ bool pair_item(const float* __restrict__ L, int64_t ldl, int R, int NE, int TOPK, int shared,
                                          int slots, int p, int* memb, int* sel, int* wp, int& e_out, int& cnt_out) {
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int r = p / slots, k = p - r * slots;
  const bool always = shared && k == TOPK;         // the shared expert: every row, slot TOPK
  constexpr int PRE = VPL <= 2 ? 2 : 1;     // rows a wave requests before the selection, to wait for them under it
  float v[PRE][VPL];
  if (!always) {
#pragma unroll
    for (int i = 0; i < PRE; ++i)
      if (wave + i * WAVES < R) topk_load<VPL>(L + (size_t)(wave + i * WAVES) * ldl, NE, lane, v[i]);
  }
  if (wave == 0) {
    int e = NE;
    if (!always) {
      float t[VPL];
      topk_load<VPL>(L + (size_t)r * ldl, NE, lane, t);
      e = topk_kth<VPL>(t, k, lane);
    }
    if (lane == 0) sel[0] = e;
  }
  __syncthreads();
  const int e = sel[0];
#pragma unroll
  for (int i = 0; i < PRE; ++i) {
    const int q = wave + i * WAVES;
    if (q >= R) break;
    int m = TOPK;
    if (!always) {
      const int slot = topk_slot_of<VPL>(v[i], e, lane);
      m = slot < TOPK ? slot : -1;
    }
    if (lane == 0) memb[q] = m;
  }
  for (int q = wave + PRE * WAVES; q < R; q += WAVES) {
    int m = TOPK;
    if (!always) {
      topk_load<VPL>(L + (size_t)q * ldl, NE, lane, v[0]);
      const int slot = topk_slot_of<VPL>(v[0], e, lane);
      m = slot < TOPK ? slot : -1;
    }
    if (lane == 0) memb[q] = m;
  }
  __syncthreads();
  const int m = lane < R ? memb[lane] : -1;
  const unsigned long long mask = __ballot(m >= 0);
  if (__popcll(mask & ((1ull << r) - 1ull)) & 1) return false;       // the second pair of an item
  const unsigned long long rest = r < 63 ? mask >> (r + 1) : 0ull;
  int p1 = p, cnt = 1;
  if (rest) {
    const int q = __builtin_amdgcn_readfirstlane(r + 1 + __builtin_ctzll(rest));
    p1 = q * slots + __builtin_amdgcn_readlane(m, q);
    cnt = 2;
  }
  wp[0] = p;
  wp[1] = p1;
  e_out = e;
  cnt_out = cnt;
  return true;
}

template <int VPL>
__device__ __forceinline__ void topk_lane_n(const float* __restrict__ row, int NE, int TOPK, int shared, int lane,
                                            int& id, float& w) {
  float v[VPL];
  topk_load<VPL>(row, NE, lane, v);
  topk_pick<VPL>(v, row, NE, TOPK, shared, lane, id, w);
}

__device__ __forceinline__ void topk_lane(const float* __restrict__ row, int NE, int TOPK, int shared, int lane,
                                          int& id, float& w) {
  if (NE <= 128) topk_lane_n<2>(row, NE, TOPK, shared, lane, id, w);
  else if (NE <= 512) topk_lane_n<8>(row, NE, TOPK, shared, lane, id, w);
  else topk_lane_n<TOPK_VPL>(row, NE, TOPK, shared, lane, id, w);
}

__device__ __forceinline__ void topk_row(const float* __restrict__ row, int NE, int TOPK, int shared, int lane,
                                         int* __restrict__ pick, float* __restrict__ wts) {
  int id;
  float w;
  topk_lane(row, NE, TOPK, shared, lane, id, w);
  if (lane < TOPK + (shared ? 1 : 0)) {
    pick[lane] = id;
    wts[lane] = w;
  }
}

// ---- plan: stable counting sort of pairs by expert -------------------------------------------------------------------

constexpr int PLAN_THREADS = 1024;
constexpr int EMAX = 1024;

// Block-wide exclusive prefix sums of three per-thread values (1024 threads = 16 waves of 64); totals in tot[3].
__device__ void scan3(int (&val)[3], int (&excl)[3], int (&tot)[3]) {
  __shared__ int wsum[3][16];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  int inc[3];
#pragma unroll
  for (int s = 0; s < 3; ++s) {
    int a = val[s];
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const int u = __shfl_up(a, o);
      if (lane >= o) a += u;
    }
    inc[s] = a;
    if (lane == 63) wsum[s][wave] = a;
  }
  __syncthreads();
#pragma unroll
  for (int s = 0; s < 3; ++s) {
    int base = 0, all = 0;
    for (int w = 0; w < 16; ++w) {
      const int t = wsum[s][w];
      if (w < wave) base += t;
      all += t;
    }
    excl[s] = base + inc[s] - val[s];
    tot[s] = all;
  }
  __syncthreads();
}

// The plan's tables of a workgroup of PLAN_THREADS threads: a thread an expert.
struct PlanLds {
  int cnt[EMAX];       // pairs of expert e
  int first[EMAX];     // its first member
  int istart[EMAX];    // its first item
};

// Whole workgroup (PLAN_THREADS threads, barriers inside); thread e brings expert e's pair count c (0 past E).
// Fills L and writes the plan's items and counts: experts ascending, an expert's pairs cut into runs of T.  The
// items are written a thread an item (an expert that holds thousands of a prompt chunk's pairs has dozens): item i
// belongs to the last expert whose first item is not past i, found by bisection of the non-decreasing istart.
__device__ void place_items(PlanLds& L, int c, int E, int T, int* __restrict__ items, int* __restrict__ counts) {
  const int tid = threadIdx.x;
  int val[3] = {c, (c + T - 1) / T, c > 0 ? 1 : 0}, excl[3], tot[3];
  scan3(val, excl, tot);
  L.cnt[tid] = c;
  L.first[tid] = excl[0];
  L.istart[tid] = excl[1];
  if (tid == 0) {
    counts[0] = tot[1];
    counts[1] = tot[2];
  }
  __syncthreads();
  for (int i = tid; i < tot[1]; i += PLAN_THREADS) {
    int lo = 0, hi = E - 1;
    while (lo < hi) {
      const int mid = (lo + hi + 1) >> 1;
      if (L.istart[mid] <= i) lo = mid;
      else hi = mid - 1;
    }
    const int j = i - L.istart[lo];
    items[3 * i] = lo;
    items[3 * i + 1] = L.first[lo] + T * j;
    items[3 * i + 2] = min(T, L.cnt[lo] - T * j);
  }
}

// One wave hands expert e's `count` pairs among pk[0 .. P) to put(rank, pair) in pair order: it walks the pairs 64 at a
// time and ranks the hits of a step with one ballot.
template <class Put>
__device__ __forceinline__ void expert_pairs(const int* pk, int P, int e, int count, int lane, Put&& put) {
  int before = 0;
  for (int p0 = 0; p0 < P && before < count; p0 += 64) {
    const int p = p0 + lane;
    const bool hit = p < P && pk[p] == e;
    const unsigned long long m = __ballot(hit);
    if (hit) put(before + __popcll(m & ((1ull << lane) - 1ull)), p);
    before += __popcll(m);
  }
}

// Inclusive prefix sums over the 64 lanes: shifts inside each row of 16 lanes through DPP, then the rows' totals
// through readlane.
__device__ __forceinline__ int wave_scan(int x) {
#define TF_SHR(V_, N_) __builtin_amdgcn_update_dpp(0, V_, 0x110 + N_, 0xf, 0xf, false)
  x += TF_SHR(x, 1);
  x += TF_SHR(x, 2);
  x += TF_SHR(x, 4);
  x += TF_SHR(x, 8);
#undef TF_SHR
  const int t0 = __builtin_amdgcn_readlane(x, 15), t1 = __builtin_amdgcn_readlane(x, 31),
            t2 = __builtin_amdgcn_readlane(x, 47);
  const int row = (threadIdx.x & 63) >> 4;
  return x + (row > 0 ? t0 : 0) + (row > 1 ? t1 : 0) + (row > 2 ? t2 : 0);
}

// ---- item descriptors ---------------------------------------------------------------------------------------------------
//
// The plan of up to PLAN_THREADS pairs by one workgroup of PLAN_THREADS threads: count, scan and place; then a wave
// an expert that has pairs collects them in pair order (ballots over the pairs, 64 a step).  pk: PLAN_THREADS ints.
__device__ __forceinline__ void plan_small(const int* __restrict__ picks, int P, int E, int T, int* __restrict__ members,
                                           int* __restrict__ items, int* __restrict__ counts, int* pk, PlanLds& plan) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  plan.cnt[tid] = 0;
  __syncthreads();
  int e = tid < P ? picks[tid] : -1;
  if ((unsigned)e >= (unsigned)E) e = -1;            // an id outside the table joins no expert (and faults nothing)
  pk[tid] = e;
  if (e >= 0) atomicAdd(&plan.cnt[e], 1);
  __syncthreads();
  place_items(plan, tid < E ? plan.cnt[tid] : 0, E, T, items, counts);
  for (int x = wave; x < E; x += PLAN_THREADS / 64) {
    const int c = plan.cnt[x], at = plan.first[x];
    if (c) expert_pairs(pk, P, x, c, lane, [&](int rank, int p) { members[at + rank] = p; });
  }
}

// What the routing kernels leave for the decode expert kernels: the plan cut again into items of at most DTILE pairs
// (a workgroup walks its rows two at a time, so short items keep every workgroup to two passes over its weights and
// spread an expert that many rows share over more workgroups).  int32 rows of DESC: row 0 holds the number of
// descriptors, row 1 + i = {expert, count, first member, 0, pairs[DTILE]}.
constexpr int DESC = 8;
constexpr int DTILE = 2;

// ---- one item of the plan, found by every workgroup for itself -----------------------------------------------------
//
// The plan orders experts ascending, an expert's pairs in pair order, in items of at most TILE.  A workgroup that knows
// every pair's expert (pk[0 .. P), in LDS) finds item `it` with a histogram, a scan over the experts by wave 0 and a
// ballot walk over the pairs: no global memory, no quadratic rank loop.

struct ItemLds {
  int cnt[EMAX];       // pairs an expert
  int sel[6];          // expert, first member, count, items in all, rank of the item's first pair in its expert, full items
  int pairs[16];
};

// Item order: every full item (TILE pairs) first, in expert order, then the experts' short last items, in expert
// order — the items that take longest start first.  Item `it` of expert e's j-th tile sits at
// it < F: (full tiles before e) + j, else F + (experts with a short tile before e), F = full items in all.
//
// Every thread of the workgroup calls this (it has barriers); pk holds P expert ids (negative = none).
// Returns false when there is no item `it`.  On return L.sel and L.pairs describe the item.
// COUNTED: the caller has already cleared L.sel, counted the pairs into L.cnt and the full tiles into L.sel[5] (as the
// loop below does) and passed a barrier.
template <int TILE, bool COUNTED = false>
__device__ __forceinline__ bool find_item(ItemLds& L, const int* pk, int P, int E, int it) {
  const int tid = threadIdx.x, threads = blockDim.x, lane = tid & 63;
  if constexpr (!COUNTED) {
    for (int e = tid; e < E; e += threads) L.cnt[e] = 0;
    if (tid < 6) L.sel[tid] = tid == 0 ? -1 : 0;
    __syncthreads();
    for (int p = tid; p < P; p += threads)
      if (pk[p] >= 0) {
        const int old = atomicAdd(&L.cnt[pk[p]], 1);
        if (old % TILE == TILE - 1) atomicAdd(&L.sel[5], 1);     // this pair completes a tile
      }
    __syncthreads();
  }
  if (tid < 64) {
    const int F = L.sel[5];
    int full_before = 0, short_before = 0, pairs_before = 0;
    for (int e0 = 0; e0 < E; e0 += 64) {
      const int e = e0 + lane, c = e < E ? L.cnt[e] : 0, f = c / TILE, r = c - TILE * f > 0 ? 1 : 0;
      const int cf = wave_scan(c | (f << 16)), ri = wave_scan(r);      // inclusive, over the 64 experts of this step
      const int ci = cf & 0xFFFF, fi = cf >> 16;
      const int first_full = full_before + fi - f;
      if (it < F ? (it >= first_full && it < first_full + f) : (r && it - F == short_before + ri - 1)) {
        const int j = it < F ? it - first_full : f;
        L.sel[0] = e;
        L.sel[1] = pairs_before + ci - c + TILE * j;
        L.sel[2] = min(TILE, c - TILE * j);
        L.sel[4] = TILE * j;
      }
      const int last = __builtin_amdgcn_readlane(cf, 63);
      full_before += last >> 16;
      pairs_before += last & 0xFFFF;
      short_before += __builtin_amdgcn_readlane(ri, 63);
    }
    if (lane == 0) L.sel[3] = full_before + short_before;
  }
  __syncthreads();
  const int e = L.sel[0];
  if (e < 0) return false;
  if (tid < 64) {
    // the expert's pairs in pair order; the item takes ranks [TILE j, TILE j + count)
    int before = 0;
    const int skip = L.sel[4], cnt = L.sel[2];
    for (int p0 = 0; p0 < P && before < skip + cnt; p0 += 64) {
      const int p = p0 + lane;
      const bool hit = p < P && pk[p] == e;
      const unsigned long long m = __ballot(hit);
      const int rank = before + __popcll(m & ((1ull << lane) - 1ull));
      if (hit && rank >= skip && rank < skip + cnt) L.pairs[rank - skip] = p;
      before += __popcll(m);
    }
  }
  __syncthreads();
  return true;
}

// pair_item with the picks given (a top-k launch ran before): pair p's expert is pick[p], the expert's pairs are
// the equal picks, in pair order, two an item.  Every wave works it out for itself from the picks alone (up to 1,024,
// all requested at once), so there is no barrier and no LDS.  An id outside [0, E) joins no item.
__device__ __forceinline__ bool pair_item_given(const int* __restrict__ pick, int P, int E, int p, int* wp, int& e_out,
                                                int& cnt_out) {
  const int lane = threadIdx.x & 63;
  int v[PLAN_THREADS / 64];
#pragma unroll
  for (int i = 0; i < PLAN_THREADS / 64; ++i) v[i] = 64 * i + lane < P ? pick[64 * i + lane] : -1;
  const int e = __builtin_amdgcn_readfirstlane(pick[p]);
  if ((unsigned)e >= (unsigned)E) return false;
  int before = 0, partner = -1;
#pragma unroll
  for (int i = 0; i < PLAN_THREADS / 64; ++i) {
    const int q0 = 64 * i;
    if (q0 >= P) break;
    const unsigned long long m = __ballot(v[i] == e);
    if (q0 + 64 <= p) {
      before += __popcll(m);
    } else if (q0 <= p) {
      const int b = p - q0;
      before += __popcll(m & ((1ull << b) - 1ull));
      const unsigned long long after = b < 63 ? m >> (b + 1) : 0ull;
      if (after) partner = p + 1 + __builtin_ctzll(after);
    } else if (m && partner < 0) {
      partner = q0 + __builtin_ctzll(m);
    }
  }
  if (before & 1) return false;       // the second pair of an item
  wp[0] = p;
  wp[1] = partner >= 0 ? partner : p;
  e_out = e;
  cnt_out = partner >= 0 ? 2 : 1;
  return true;
}

}  // namespace
}  // namespace tf
