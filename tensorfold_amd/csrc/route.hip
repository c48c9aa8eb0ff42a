// MoE glue around the expert kernels: router logits, per-row top-k, the stable grouping of pairs by expert, and the
// weighted combine.  All integer results (ids, members, items) are deterministic and independent of the row count.

#include "routing.h"

namespace tf {
namespace {

// ---- router: logits[m, e] = x[m] . rows[e], bf16 MFMA, K in steps of 32 in order ------------------------------------

__global__ void __launch_bounds__(64)
    router_kernel(const uint16_t* __restrict__ X, int64_t ldx, const uint16_t* __restrict__ R, float* __restrict__ out,
                  int M, int D, int NE) {
  const int lane = threadIdx.x, r = lane & 15, kq = lane >> 4;
  const int m0 = blockIdx.x * 16, e0 = blockIdx.y * 16;
  const uint16_t* xa = X + (size_t)min(m0 + r, M - 1) * ldx + kq * 8;
  const uint16_t* wb = R + (size_t)min(e0 + r, NE - 1) * D + kq * 8;
  f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
  for (int k0 = 0; k0 < D; k0 += 32) {
    const bf16x8_t a = *reinterpret_cast<const bf16x8_t*>(xa + k0);
    const bf16x8_t b = *reinterpret_cast<const bf16x8_t*>(wb + k0);
    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc, 0, 0, 0);
  }
  const int col = e0 + r;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int row = m0 + 4 * kq + i;
    if (row < M && col < NE) out[(size_t)row * NE + col] = acc[i];
  }
}

__global__ void __launch_bounds__(64)
    topk_kernel(const float* __restrict__ L, int64_t ldl, int NE, int TOPK, int shared, int* __restrict__ pick,
                float* __restrict__ wts) {
  const int r = blockIdx.x, slots = TOPK + (shared ? 1 : 0);
  topk_row(L + (size_t)r * ldl, NE, TOPK, shared, threadIdx.x, pick + (size_t)r * slots, wts + (size_t)r * slots);
}

// ---- plan: stable counting sort of pairs by expert -------------------------------------------------------------------

// up to 1024 pairs: one workgroup counts, scans and places; then a wave an expert that has pairs collects them in
// pair order (ballots over the pairs, 64 a step)
__global__ void __launch_bounds__(PLAN_THREADS)
    plan_small_kernel(const int* __restrict__ picks, int P, int E, int T, int* __restrict__ members,
                      int* __restrict__ items, int* __restrict__ counts) {
  __shared__ int pk[PLAN_THREADS];
  __shared__ PlanLds plan;
  plan_small(picks, P, E, T, members, items, counts, pk, plan);
}

// The decode layer's whole routing in one workgroup (rows * slots <= 1024): top-k of every row, the pair sort, one
// descriptor an item for the fused expert kernel {expert, count, first, 0, pairs[16]}, and the zeroing of the fused
// kernel's counters.

__global__ void __launch_bounds__(PLAN_THREADS)
    route_decode_kernel(const float* __restrict__ L, int64_t ldl, int R, int NE, int TOPK, int shared,
                        int* __restrict__ pick, float* __restrict__ wts, int* __restrict__ members,
                        int* __restrict__ items, int* __restrict__ counts, int* __restrict__ desc,
                        int* __restrict__ zero, int n_zero, int have_picks) {
  __shared__ int pk[PLAN_THREADS];
  __shared__ PlanLds plan;
  __shared__ int mem[PLAN_THREADS];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int slots = TOPK + (shared ? 1 : 0), P = R * slots, E = NE + (shared ? 1 : 0), T = 16;
  plan.cnt[tid] = 0;
  for (int i = tid; i < n_zero; i += PLAN_THREADS) zero[i] = 0;
  if (!have_picks) {      // else a launch before this one has left the picks and the weights
    for (int r = wave; r < R; r += PLAN_THREADS / 64)
      topk_row(L + (size_t)r * ldl, NE, TOPK, shared, lane, pick + (size_t)r * slots, wts + (size_t)r * slots);
  }
  __threadfence_block();
  __syncthreads();
  int e = tid < P ? pick[tid] : -1;
  if ((unsigned)e >= (unsigned)E) e = -1;
  pk[tid] = e;
  if (e >= 0) atomicAdd(&plan.cnt[e], 1);
  __syncthreads();
  place_items(plan, tid < E ? plan.cnt[tid] : 0, E, T, items, counts);
  for (int x = wave; x < E; x += PLAN_THREADS / 64) {
    const int c = plan.cnt[x], at = plan.first[x];
    if (c)
      expert_pairs(pk, P, x, c, lane, [&](int rank, int p) {
        members[at + rank] = p;
        mem[at + rank] = p;
      });
  }
  __threadfence_block();
  __syncthreads();
  const int* cnt = plan.cnt;
  const int* off = plan.first;
  // the descriptors: the same members cut into items of DTILE, every full item first (they take longest), then the
  // experts' short last items
  const int c = tid < E ? cnt[tid] : 0, f = c / DTILE, r = c - DTILE * f > 0 ? 1 : 0;
  int val[3] = {f, r, 0}, excl[3], tot[3];
  scan3(val, excl, tot);
  if (tid == 0) desc[0] = tot[0] + tot[1];
  for (int j = 0; j < f + r; ++j) {
    int* d = desc + (size_t)(1 + (j < f ? excl[0] + j : tot[0] + excl[1])) * DESC;
    const int first = off[tid] + DTILE * j, n = min(DTILE, c - DTILE * j);
    d[0] = tid;
    d[1] = n;
    d[2] = first;
    d[3] = 0;
    for (int k = 0; k < DTILE; ++k) d[4 + k] = k < n ? mem[first + k] : 0;
  }
}

// wide plans, pass 1: block b ranks its 1024 pairs within each expert (pair order) and leaves its counts in hist[b].
// A pair's rank = the pairs of its expert in earlier waves of the block + those in earlier lanes of its wave: the
// lanes are compared through 64 readlanes, the waves' counts (one writer each: the expert's last lane in the wave)
// are prefixed by a thread an expert.
__global__ void __launch_bounds__(PLAN_THREADS)
    plan_rank_kernel(const int* __restrict__ picks, int P, int E, int* __restrict__ rank, int* __restrict__ hist) {
  constexpr int NW = PLAN_THREADS / 64;
  __shared__ unsigned short wcnt[NW][EMAX];      // pairs of expert e in wave w; then: in the waves before w
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, p = blockIdx.x * PLAN_THREADS + tid;
  for (int i = tid; i < NW * EMAX; i += PLAN_THREADS) (&wcnt[0][0])[i] = 0;
  int e = -1;
  if (p < P) {
    e = picks[p];
    if ((unsigned)e >= (unsigned)E) e = -1;
  }
  int before = 0, later = 0;
  for (int l = 0; l < 64; ++l) {
    const int el = __builtin_amdgcn_readlane(e, l);
    before += (l < lane) & (el == e);
    later |= (l > lane) & (el == e);
  }
  __syncthreads();
  if (e >= 0 && !later) wcnt[wave][e] = (unsigned short)(before + 1);
  __syncthreads();
  if (tid < E) {
    int acc = 0;
#pragma unroll
    for (int w = 0; w < NW; ++w) {
      const int c = wcnt[w][tid];
      wcnt[w][tid] = (unsigned short)acc;
      acc += c;
    }
    hist[(size_t)blockIdx.x * E + tid] = acc;
  }
  __syncthreads();
  if (e >= 0) rank[p] = wcnt[wave][e] + before;
}

// pass 2, one block: hist[b][e] becomes block b's first member of expert e; items and counts are written
__global__ void __launch_bounds__(PLAN_THREADS)
    plan_offsets_kernel(int nblk, int E, int T, int* __restrict__ hist, int* __restrict__ items,
                        int* __restrict__ counts) {
  const int tid = threadIdx.x;
  constexpr int CH = 16;             // blocks read together: independent loads, one trip through memory a chunk
  int c = 0;
  if (tid < E)
    for (int b0 = 0; b0 < nblk; b0 += CH) {
      int v[CH];
#pragma unroll
      for (int i = 0; i < CH; ++i) v[i] = b0 + i < nblk ? hist[(size_t)(b0 + i) * E + tid] : 0;
#pragma unroll
      for (int i = 0; i < CH; ++i) c += v[i];
    }
  __shared__ PlanLds plan;
  place_items(plan, c, E, T, items, counts);
  int run = plan.first[tid];
  if (tid < E)
    for (int b0 = 0; b0 < nblk; b0 += CH) {
      int v[CH];
#pragma unroll
      for (int i = 0; i < CH; ++i) v[i] = b0 + i < nblk ? hist[(size_t)(b0 + i) * E + tid] : 0;
#pragma unroll
      for (int i = 0; i < CH; ++i)
        if (b0 + i < nblk) {
          hist[(size_t)(b0 + i) * E + tid] = run;
          run += v[i];
        }
    }
}

// pass 3: every pair to its place
__global__ void plan_scatter_kernel(const int* __restrict__ picks, int P, int E, const int* __restrict__ rank,
                                    const int* __restrict__ hist, int* __restrict__ members) {
  const int p = blockIdx.x * blockDim.x + threadIdx.x;
  if (p >= P) return;
  const int e = picks[p];
  if ((unsigned)e < (unsigned)E) members[hist[(size_t)(p / PLAN_THREADS) * E + e] + rank[p]] = p;
}

// ---- combine ---------------------------------------------------------------------------------------------------------

// YKIND: what the pair outputs are stored as: 0 fp32, 1 bf16, 2 fp16
template <int YKIND>
__global__ void __launch_bounds__(256)
    combine_kernel(const void* __restrict__ Y, const float* __restrict__ Wt, uint16_t* __restrict__ out, int S, int D) {
  const int r = blockIdx.x;
  const int d = (blockIdx.y * 256 + threadIdx.x) * 2;
  if (d >= D) return;
  float a0 = 0.f, a1 = 0.f;
  // eight slots' loads go out together, then the sum in slot order
  for (int k0 = 0; k0 < S; k0 += 8) {
    float w[8], v0[8], v1[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int k = k0 + j < S ? k0 + j : S - 1;
      w[j] = Wt[(size_t)r * S + k];
      const size_t at = ((size_t)r * S + k) * D + d;
      if (YKIND == 1) {
        const uint32_t v = *reinterpret_cast<const uint32_t*>(reinterpret_cast<const uint16_t*>(Y) + at);
        v0[j] = bf16_lo(v);
        v1[j] = bf16_hi(v);
      } else if (YKIND == 2) {
        typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
        const half2_t v = *reinterpret_cast<const half2_t*>(reinterpret_cast<const _Float16*>(Y) + at);
        v0[j] = (float)v[0];
        v1[j] = (float)v[1];
      } else {
        const float2 v = *reinterpret_cast<const float2*>(reinterpret_cast<const float*>(Y) + at);
        v0[j] = v.x;
        v1[j] = v.y;
      }
    }
#pragma unroll
    for (int j = 0; j < 8; ++j)
      if (k0 + j < S) {
        a0 = fmaf(w[j], v0[j], a0);
        a1 = fmaf(w[j], v1[j], a1);
      }
  }
  *reinterpret_cast<uint32_t*>(out + (size_t)r * D + d) = pack_bf16(a0, a1);
}

// fp32 pair outputs, four columns a thread (16-byte loads): the wide prompt chunks, where the combine is a 370 MB read
__global__ void __launch_bounds__(256)
    combine4_kernel(const float* __restrict__ Y, const float* __restrict__ Wt, uint16_t* __restrict__ out, int S, int D) {
  const int r = blockIdx.x;
  const int d = (blockIdx.y * 256 + threadIdx.x) * 4;
  if (d >= D) return;
  float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
  const float* y = Y + (size_t)r * S * D + d;
  for (int k0 = 0; k0 < S; k0 += 8) {
    float w[8];
    f32x4_t v[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int k = k0 + j < S ? k0 + j : S - 1;
      w[j] = Wt[(size_t)r * S + k];
      v[j] = __builtin_nontemporal_load(reinterpret_cast<const f32x4_t*>(y + (size_t)k * D));
    }
#pragma unroll
    for (int j = 0; j < 8; ++j)
      if (k0 + j < S) {
        a0 = fmaf(w[j], v[j][0], a0);
        a1 = fmaf(w[j], v[j][1], a1);
        a2 = fmaf(w[j], v[j][2], a2);
        a3 = fmaf(w[j], v[j][3], a3);
      }
  }
  *reinterpret_cast<uint2*>(out + (size_t)r * D + d) = make_uint2(pack_bf16(a0, a1), pack_bf16(a2, a3));
}

}  // namespace
}  // namespace tf

using namespace tf;

extern "C" int tf_moe_router(const uint16_t* x, int64_t ldx, const uint16_t* rows, float* logits, int m, int d, int ne,
                             tf_stream_t stream) {
  clear_error();
  TF_REQUIRE(x && rows && logits && m >= 1 && ne >= 1, "router: null pointer or empty shape");
  TF_REQUIRE(d >= 32 && d % 32 == 0, "router: the hidden size (%d) must be a multiple of 32", d);
  TF_REQUIRE(aligned16(x) && aligned16(rows) && ldx % 8 == 0, "router: x and rows must be 16-byte aligned");
  router_kernel<<<dim3((m + 15) / 16, (ne + 15) / 16), 64, 0, as_stream(stream)>>>(x, ldx, rows, logits, m, d, ne);
  TF_LAUNCH_OK("tf_moe_router");
  return 0;
}

extern "C" int tf_moe_topk(const float* logits, int64_t ldl, int rows, int experts, int top_k, int shared,
                           int32_t* pick, float* wts, tf_stream_t stream) {
  clear_error();
  TF_REQUIRE(logits && pick && wts && rows >= 1, "topk: null pointer or empty shape");
  TF_REQUIRE(experts >= 1 && experts <= 64 * TOPK_VPL, "topk: 1 to %d experts, not %d", 64 * TOPK_VPL, experts);
  TF_REQUIRE(top_k >= 1 && top_k + (shared ? 1 : 0) <= 64 && top_k <= experts, "topk: 1 to 64 slots a row, not %d", top_k);
  TF_REQUIRE(ldl >= experts + (shared ? 1 : 0), "topk: logits rows hold %lld values, %d are read", (long long)ldl,
             experts + (shared ? 1 : 0));
  topk_kernel<<<rows, 64, 0, as_stream(stream)>>>(logits, ldl, experts, top_k, shared, pick, wts);
  TF_LAUNCH_OK("tf_moe_topk");
  return 0;
}

extern "C" int tf_moe_route_decode(const float* logits, int64_t ldl, int rows, int experts, int top_k, int shared,
                                   int32_t* pick, float* wts, int32_t* members, int32_t* items, int32_t* counts,
                                   int32_t* desc, int32_t* zero, int n_zero, tf_stream_t stream) {
  clear_error();
  TF_REQUIRE(logits && pick && wts && members && items && counts && desc, "route: null pointer argument");
  TF_REQUIRE(experts >= 1 && experts + (shared ? 1 : 0) <= EMAX && experts <= 64 * TOPK_VPL,
             "route: at most %d experts", EMAX - 1);
  TF_REQUIRE(top_k >= 1 && top_k + (shared ? 1 : 0) <= 64 && top_k <= experts, "route: 1 to 64 slots a row, not %d", top_k);
  TF_REQUIRE(rows >= 1 && (int64_t)rows * (top_k + (shared ? 1 : 0)) <= PLAN_THREADS,
             "route: the fused decode routing takes at most %d pairs", PLAN_THREADS);
  TF_REQUIRE(ldl >= experts + (shared ? 1 : 0), "route: logits rows are too short");
  TF_REQUIRE(n_zero >= 0 && (n_zero == 0 || zero), "route: bad counter range");
  // more rows than the one workgroup has waves: the top-k runs first, a workgroup a row, spread over the chip
  const int spread = rows > PLAN_THREADS / 64;
  if (spread) topk_kernel<<<rows, 64, 0, as_stream(stream)>>>(logits, ldl, experts, top_k, shared, pick, wts);
  route_decode_kernel<<<1, PLAN_THREADS, 0, as_stream(stream)>>>(logits, ldl, rows, experts, top_k, shared, pick, wts,
                                                                members, items, counts, desc, zero, n_zero, spread);
  TF_LAUNCH_OK("tf_moe_route_decode");
  return 0;
}

extern "C" int tf_experts_plan(const int32_t* picks, int64_t pairs, int experts, int tile, int32_t* members,
                               int32_t* items, int32_t* counts, int32_t* rank, int32_t* hist, tf_stream_t stream) {
  clear_error();
  TF_REQUIRE(picks && members && items && counts, "plan: null pointer argument");
  TF_REQUIRE(experts >= 1 && experts <= EMAX, "experts: at most %d experts", EMAX);
  TF_REQUIRE(tile == 16 || tile == 64 || tile == 128, "items hold 16 pairs (decode) or 64 or 128 (prefill)");
  TF_REQUIRE(pairs >= 0 && pairs <= 0x7FFFFFFF, "plan: pair count out of range");
  hipStream_t s = as_stream(stream);
  const int P = (int)pairs;
  if (P <= PLAN_THREADS) {
    plan_small_kernel<<<1, PLAN_THREADS, 0, s>>>(picks, P, experts, tile, members, items, counts);
    TF_LAUNCH_OK("tf_experts_plan");
    return 0;
  }
  TF_REQUIRE(rank && hist, "experts: plan scratch (rank, hist) is needed past %d pairs", PLAN_THREADS);
  const int nblk = (P + PLAN_THREADS - 1) / PLAN_THREADS;
  plan_rank_kernel<<<nblk, PLAN_THREADS, 0, s>>>(picks, P, experts, rank, hist);
  plan_offsets_kernel<<<1, PLAN_THREADS, 0, s>>>(nblk, experts, tile, hist, items, counts);
  plan_scatter_kernel<<<(P + 255) / 256, 256, 0, s>>>(picks, P, experts, rank, hist, members);
  TF_LAUNCH_OK("tf_experts_plan");
  return 0;
}

extern "C" int tf_moe_combine(const void* y, int y_bf16, const float* wts, uint16_t* out, int rows, int slots, int d,
                              tf_stream_t stream) {
  clear_error();
  TF_REQUIRE(y && wts && out && rows >= 1 && slots >= 1, "combine: null pointer or empty shape");
  TF_REQUIRE(d >= 2 && d % 2 == 0, "combine: the hidden size (%d) must be even", d);
  if (!y_bf16 && d % 4 == 0 && aligned16(y) && rows >= 64) {
    combine4_kernel<<<dim3(rows, (d / 4 + 255) / 256), 256, 0, as_stream(stream)>>>(
        static_cast<const float*>(y), wts, out, slots, d);
    TF_LAUNCH_OK("tf_moe_combine");
    return 0;
  }
  const dim3 grid(rows, (d / 2 + 255) / 256);
  if (y_bf16 == 1) combine_kernel<1><<<grid, 256, 0, as_stream(stream)>>>(y, wts, out, slots, d);
  else if (y_bf16 == 2) combine_kernel<2><<<grid, 256, 0, as_stream(stream)>>>(y, wts, out, slots, d);
  else combine_kernel<0><<<grid, 256, 0, as_stream(stream)>>>(y, wts, out, slots, d);
  TF_LAUNCH_OK("tf_moe_combine");
  return 0;
}
