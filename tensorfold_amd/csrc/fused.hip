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

namespace tf {
namespace {

constexpr int DESC = 20;      // int32 an item descriptor: expert, count, first, 0, pairs[16]

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

template <int GS, int NM, int EPI_UP, int WAVES>
__global__ void __launch_bounds__(WAVES * 64)
    moe_fused_kernel(const uint16_t* __restrict__ X, int64_t x_stride, int slots, const uint32_t* __restrict__ Wup,
                     const uint32_t* __restrict__ Wdown, int D, int NI, const int* __restrict__ desc,
                     const int* __restrict__ counts, const float* __restrict__ wts, const float* __restrict__ xs_x,
                     uint16_t* __restrict__ act, float* __restrict__ xs_act, float* __restrict__ y,
                     uint16_t* __restrict__ out, int* __restrict__ done, int* __restrict__ arrive,
                     int* __restrict__ status, float limit, int max_items, int spins) {
  extern __shared__ float lds[];
  __shared__ int pairs[16];
  __shared__ int last[16];
  const int NB2u = (NI / 32 + 1) >> 1, NB2d = (D / 32 + 1) >> 1;
  const int U = max_items * NB2u;
  const int b = blockIdx.x, tid = threadIdx.x;
  const bool up = b < U;
  const int it = up ? b / NB2u : (b - U) / NB2d;
  const int cb2 = up ? b - it * NB2u : (b - U) - it * NB2d;
  if (it >= counts[0]) return;
  const int* d = desc + (size_t)it * DESC;
  const int e = d[0], cnt = d[1];
  if (tid < 16) pairs[tid] = d[4 + tid];
  __syncthreads();
  if (up) {
    NoHook none;
    expert_unit<GS, NM, EPI_UP, WAVES, true, COH_OUT>(X, x_stride, slots, Wup, D / GS, NI / 32, e, cnt, pairs, cb2, act,
                                                      NI, limit, xs_x, xs_act, lds, none);
    __builtin_amdgcn_s_waitcnt(0);      // every store of this wave is acknowledged ...
    __syncthreads();                    // ... of every wave ...
    if (tid == 0) __hip_atomic_fetch_add(done + it, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // ... then it counts
    return;
  }
  WaitItem wait{done + it, NB2u, spins, status};
  constexpr int DCOH = COH_IN | COH_OUT;
  if (!expert_unit<GS, 1, 0, WAVES, true, DCOH>(act, NI, 0, Wdown, NI / GS, D / 32, e, cnt, pairs, cb2, y, D,
                                                            0.f, xs_act, nullptr, lds, wait))
    return;                     // the wait ran out: status is set, nothing is published
  // this unit's 64 columns of y are written for its rows: count it in each row's token; the last one combines
  __builtin_amdgcn_s_waitcnt(0);
  __syncthreads();
  if (tid < cnt) {
    const int token = pairs[tid] / slots;
    last[tid] = __hip_atomic_fetch_add(arrive + (size_t)token * NB2d + cb2, 1, __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_AGENT) == slots - 1;
  }
  __syncthreads();
  const int lane = tid & 63, wave = tid >> 6;
  const int col = cb2 * 64 + lane;
  for (int r = wave; r < cnt; r += WAVES) {
    if (!last[r] || col >= D) continue;
    const int token = pairs[r] / slots;
    float a = 0.f;
    for (int k = 0; k < slots; ++k) {
      const float w = wts[(size_t)token * slots + k];
      a = fmaf(w, ld_agent(y + ((size_t)token * slots + k) * D + col), a);
    }
    out[(size_t)token * D + col] = (uint16_t)f32_bf16_bits(a);
  }
}

int fused_waves(int64_t grid) { return grid < 768 ? 16 : grid < 1536 ? 8 : 4; }

template <int GS, int NM, int EPI_UP>
int launch_fused(const uint16_t* x, int64_t x_stride, int slots, const uint32_t* wup, const uint32_t* wdown, int d,
                 int ni, const int* desc, const int* counts, const float* wts, const float* xs_x, uint16_t* act,
                 float* xs_act, float* y, uint16_t* out, int* done, int* arrive, int* status, float limit,
                 int max_items, hipStream_t stream) {
  const int nb2u = (ni / 32 + 1) / 2, nb2d = (d / 32 + 1) / 2;
  const int64_t grid = (int64_t)max_items * (nb2u + nb2d);
  if (grid < 1) return 0;
  TF_REQUIRE(grid <= 0x7FFFFFFF, "moe: %lld workgroups exceed the grid limit", (long long)grid);
  const size_t smem = sizeof(float) * expert_lds_floats(NM, 0, true);
  const int spins = 1 << 16;     // polls of about a microsecond: far past any real wait, short enough to drain fast
  const dim3 g((unsigned)grid);
#define TF_GO(W_)                                                                                                 \
  moe_fused_kernel<GS, NM, EPI_UP, W_><<<g, W_ * 64, smem, stream>>>(x, x_stride, slots, wup, wdown, d, ni, desc, \
                                                                     counts, wts, xs_x, act, xs_act, y, out, done, \
                                                                     arrive, status, limit, max_items, spins)
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

extern "C" int tf_moe_decode_experts(int gs, int swiglu, const uint16_t* x, int64_t x_stride, int rows, int slots,
                                     const uint32_t* up, const uint32_t* down, int d, int ni, const int32_t* desc,
                                     const int32_t* counts, const float* wts, const float* xs_x, uint16_t* act,
                                     float* xs_act, float* y, uint16_t* out, int32_t* done, int32_t* arrive,
                                     int32_t* status, float limit, int max_items, tf_stream_t stream) {
  clear_error();
  TF_REQUIRE(gs == 32 || gs == 64, "moe: groups of 32 or 64 inputs, not %d", gs);
  TF_REQUIRE(x && up && down && desc && counts && wts && xs_x && act && xs_act && y && out && done && arrive && status,
             "moe: null pointer argument");
  TF_REQUIRE(d % 64 == 0 && ni % 64 == 0 && d % gs == 0 && ni % gs == 0,
             "moe: the fused decode layer takes hidden and intermediate sizes that are multiples of 64");
  TF_REQUIRE(aligned16(x) && x_stride % 8 == 0 && aligned16(up) && aligned16(down) && aligned16(act),
             "x: rows of K = groups * group size inputs, 16-byte aligned");
  TF_REQUIRE(rows >= 1 && slots >= 1 && max_items >= 1, "moe: empty call");
  hipStream_t s = as_stream(stream);
  if (gs == 64)
    return swiglu ? launch_fused<64, 2, 2>(x, x_stride, slots, up, down, d, ni, desc, counts, wts, xs_x, act, xs_act, y,
                                           out, done, arrive, status, limit, max_items, s)
                  : launch_fused<64, 1, 1>(x, x_stride, slots, up, down, d, ni, desc, counts, wts, xs_x, act, xs_act, y,
                                           out, done, arrive, status, limit, max_items, s);
  return swiglu ? launch_fused<32, 2, 2>(x, x_stride, slots, up, down, d, ni, desc, counts, wts, xs_x, act, xs_act, y,
                                         out, done, arrive, status, limit, max_items, s)
                : launch_fused<32, 1, 1>(x, x_stride, slots, up, down, d, ni, desc, counts, wts, xs_x, act, xs_act, y,
                                         out, done, arrive, status, limit, max_items, s);
}
