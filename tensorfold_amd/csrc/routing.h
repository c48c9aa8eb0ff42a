// Routing pieces shared by the routing kernels and the decode kernels that route for themselves: the per-row top-k
// (one wave a row), block-wide scans, and the lookup of one item of the pair sort without building the whole plan.
#pragma once

#include "tf_common.h"

namespace tf {
namespace {

// ---- top-k: one wave a row ------------------------------------------------------------------------------------------

constexpr int TOPK_VPL = 16;     // values a lane: up to 1024 experts

// one wave, one row (see tf_moe_topk): lane k < TOPK leaves with the k-th pick and its weight, lane TOPK with the
// shared expert's when there is one
__device__ __forceinline__ void topk_lane(const float* __restrict__ row, int NE, int TOPK, int shared, int lane,
                                          int& id, float& w) {
  const float NEG = -__builtin_inff();
  float v[TOPK_VPL];
#pragma unroll
  for (int i = 0; i < TOPK_VPL; ++i) {
    const int e = lane + 64 * i;
    v[i] = e < NE ? row[e] : NEG;
  }
  float top = 0.f, total = 0.f, mine_ex = 0.f;
  int mine_id = 0;
  for (int k = 0; k < TOPK; ++k) {
    float bv = v[0];
    int bi = lane;
#pragma unroll
    for (int i = 1; i < TOPK_VPL; ++i)
      if (v[i] > bv) {
        bv = v[i];
        bi = lane + 64 * i;
      }
    float m = bv;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o));
    int idx = bv == m ? bi : 0x7FFFFFFF;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) idx = min(idx, __shfl_xor(idx, o));
    if (k == 0) top = m;
    const float ex = expf(m - top);
    total += ex;
    if (lane == k) {
      mine_ex = ex;
      mine_id = idx;
    }
    if ((idx & 63) == lane) {
#pragma unroll
      for (int i = 0; i < TOPK_VPL; ++i)
        if (i == (idx >> 6)) v[i] = NEG;
    }
  }
  id = mine_id;
  w = round_bf16(mine_ex / total);
  if (shared && lane == TOPK) {
    const float sg = round_bf16(row[NE]);
    id = NE;
    w = round_bf16(1.f / (1.f + expf(-sg)));
  }
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

// thread e: expert e's pair count c -> its first member; writes the items (expert order) and counts
__device__ int place_items(int c, int E, int T, int* __restrict__ items, int* __restrict__ counts) {
  const int tid = threadIdx.x;
  const int tiles = (c + T - 1) / T;
  int val[3] = {c, tiles, c > 0 ? 1 : 0}, excl[3], tot[3];
  scan3(val, excl, tot);
  if (tid == 0) {
    counts[0] = tot[1];
    counts[1] = tot[2];
  }
  if (tid < E)
    for (int j = 0; j < tiles; ++j) {
      int* it = items + 3 * (excl[1] + j);
      it[0] = tid;
      it[1] = excl[0] + T * j;
      it[2] = min(T, c - T * j);
    }
  return excl[0];
}

// ---- one item of the plan, found by every workgroup for itself -----------------------------------------------------
//
// The plan orders experts ascending, an expert's pairs in pair order, in items of at most 16.  A workgroup that knows
// every pair's expert (pk[0 .. P), in LDS) finds item `it` with a histogram, a scan over the experts by wave 0 and a
// ballot walk over the pairs: no global memory, no quadratic rank loop.

struct ItemLds {
  int cnt[EMAX];       // pairs an expert
  int sel[5];          // expert, first member, count, items in all, rank of the item's first pair in its expert
  int pairs[16];
};

// Every thread of the workgroup calls this (it has barriers); pk holds P expert ids (negative = none).
// Returns false when there is no item `it`.  On return L.sel and L.pairs describe the item.
__device__ __forceinline__ bool find_item(ItemLds& L, const int* pk, int P, int E, int it) {
  const int tid = threadIdx.x, threads = blockDim.x, lane = tid & 63;
  for (int e = tid; e < E; e += threads) L.cnt[e] = 0;
  if (tid < 5) L.sel[tid] = tid == 0 ? -1 : 0;
  __syncthreads();
  for (int p = tid; p < P; p += threads)
    if (pk[p] >= 0) atomicAdd(&L.cnt[pk[p]], 1);
  __syncthreads();
  if (tid < 64) {
    int items_before = 0, pairs_before = 0;
    for (int e0 = 0; e0 < E; e0 += 64) {
      const int e = e0 + lane, c = e < E ? L.cnt[e] : 0, t = (c + 15) >> 4;
      int ti = t, ci = c;                        // inclusive scans over the 64 experts of this step
#pragma unroll
      for (int o = 1; o < 64; o <<= 1) {
        const int ut = __shfl_up(ti, o), uc = __shfl_up(ci, o);
        if (lane >= o) {
          ti += ut;
          ci += uc;
        }
      }
      const int first_item = items_before + ti - t;
      if (it >= first_item && it < first_item + t) {
        const int j = it - first_item;
        L.sel[0] = e;
        L.sel[1] = pairs_before + ci - c + 16 * j;
        L.sel[2] = min(16, c - 16 * j);
        L.sel[4] = 16 * j;
      }
      items_before += __shfl(ti, 63);
      pairs_before += __shfl(ci, 63);
    }
    if (lane == 0) L.sel[3] = items_before;
  }
  __syncthreads();
  const int e = L.sel[0];
  if (e < 0) return false;
  if (tid < 64) {
    // the expert's pairs in pair order; the item takes ranks [16 j, 16 j + count)
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

}  // namespace
}  // namespace tf
