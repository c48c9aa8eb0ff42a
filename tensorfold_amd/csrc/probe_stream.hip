// What one launch can stream with the decode expert units' own access pattern and nothing else: the ceiling the decode
// kernels are measured against beside the 8 TB/s peak.  A workgroup takes one unit of benchmark configuration 1's up
// projection (two 32-column blocks of one expert: 42 groups of 64 inputs, 1,152 bytes a block and group: 1,024 of codes
// and 128 of scale | bias); its waves split the groups as the kernels split their K slices; a lane loads what the
// kernels' lanes load (two 16-byte pieces and one dword a group, two groups in flight) and only XORs it.  Variants:
// the unit's index read through two dependent loads first (a descriptor, then the item), units laid one after the
// other or scattered over 41 of 128 experts' tables as a routing draw scatters them.  Launches run back to back on
// one stream over four tables of 359 MB, so every launch reads HBM.  A stand-alone program: `python bench_configs.py
// floor` runs the binary that tensorfold_amd/build.py compiled beside the library.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdio>
#include <vector>

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
constexpr int KG = 42, BW = 288, UNITS_AN_EXPERT = 29, EXPERTS = 128, DRAWS = 64;

#define CK(X_)                                                                    \
  do {                                                                            \
    hipError_t e_ = (X_);                                                         \
    if (e_ != hipSuccess) {                                                       \
      std::printf("probe_stream: %s at line %d\n", hipGetErrorString(e_), __LINE__); \
      return 1;                                                                   \
    }                                                                             \
  } while (0)

template <int WAVES, bool SCATTER>
__global__ void __launch_bounds__(WAVES * 64)
    unit_kernel(const unsigned* __restrict__ W, const int* __restrict__ chain, const int* __restrict__ draws, int draw,
                unsigned* sink) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int unit = chain[4096 + chain[blockIdx.x]];          // two trips before the first weight is requested
  if (SCATTER) unit = draws[draw * DRAWS + unit / UNITS_AN_EXPERT] * UNITS_AN_EXPERT + unit % UNITS_AN_EXPERT;
  const unsigned* base = W + ((size_t)(2 * unit + (lane >> 5)) * KG) * BW + (lane & 31) * 4;
  const int gA = wave * KG / WAVES, gB = (wave + 1) * KG / WAVES;
  u32x4 acc = {0, 0, 0, 0};
  unsigned sacc = 0;
  u32x4 v[2][2];
  unsigned sb[2];
  auto load = [&](int d, int g) {
    const unsigned* p = base + (size_t)g * BW;
    v[d][0] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
    v[d][1] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p + 128));
    sb[d] = __builtin_nontemporal_load(p - (lane & 31) * 4 + 256 + (lane & 31));
  };
#pragma unroll
  for (int d = 0; d < 2; ++d)
    if (gA + d < gB) load(d, gA + d);
  for (int g0 = gA; g0 < gB; g0 += 2) {
#pragma unroll
    for (int d = 0; d < 2; ++d) {
      const int g = g0 + d;
      if (g < gB) {
        acc ^= v[d][0] ^ v[d][1];
        sacc ^= sb[d];
        if (g + 2 < gB) load(d, g + 2);
      }
    }
  }
  if ((acc.x ^ acc.y ^ acc.z ^ acc.w ^ sacc) == 0x12345678u) sink[0] = 1;
}

int main() {
  const int NBUF = 4;
  const size_t unit_bytes = (size_t)2 * KG * BW * 4, table = unit_bytes * EXPERTS * UNITS_AN_EXPERT;
  std::vector<void*> bufs(NBUF);
  for (auto& b : bufs) {
    CK(hipMalloc(&b, table));
    CK(hipMemset(b, 1, table));
  }
  std::vector<int> chain(8192), draws(DRAWS * DRAWS);
  for (int i = 0; i < 4096; ++i) chain[i] = chain[4096 + i] = i;
  unsigned rng = 12345;
  for (int d = 0; d < DRAWS; ++d) {          // a draw: 41 distinct experts of 128, in expert order as a plan lists them
    std::vector<int> all(EXPERTS);
    for (int i = 0; i < EXPERTS; ++i) all[i] = i;
    for (int i = 0; i < 41; ++i) {
      rng = rng * 1664525u + 1013904223u;
      std::swap(all[i], all[i + (rng >> 8) % (EXPERTS - i)]);
    }
    std::sort(all.begin(), all.begin() + 41);
    for (int i = 0; i < DRAWS; ++i) draws[d * DRAWS + i] = all[i % 41];
  }
  int *dchain, *ddraws;
  unsigned* sink;
  CK(hipMalloc(&dchain, chain.size() * 4));
  CK(hipMalloc(&ddraws, draws.size() * 4));
  CK(hipMalloc(&sink, 4));
  CK(hipMemcpy(dchain, chain.data(), chain.size() * 4, hipMemcpyHostToDevice));
  CK(hipMemcpy(ddraws, draws.data(), draws.size() * 4, hipMemcpyHostToDevice));
  hipEvent_t a, b;
  hipStream_t s;
  CK(hipEventCreate(&a));
  CK(hipEventCreate(&b));
  CK(hipStreamCreate(&s));
  std::printf("units (tokens of configuration 1)  waves  layout      MB      us    TB/s\n");
  for (int units : {174, 638, 1172}) {          // 6, 22 and 40.4 experts' units: 1, 4 and 8 tokens
    const double mb = units * (double)unit_bytes * 1e-6;
#define TF_RUN(W_, SC_)                                                                                         \
  {                                                                                                             \
    auto launch = [&](int i) {                                                                                  \
      unit_kernel<W_, SC_><<<units, W_ * 64, 0, s>>>((const unsigned*)bufs[i % NBUF], dchain, ddraws, i % DRAWS, sink); \
    };                                                                                                          \
    for (int i = 0; i < NBUF; ++i) launch(i);                                                                   \
    CK(hipStreamSynchronize(s));                                                                                \
    const int reps = 80;                                                                                        \
    CK(hipEventRecord(a, s));                                                                                   \
    for (int i = 0; i < reps; ++i) launch(i);                                                                   \
    CK(hipEventRecord(b, s));                                                                                   \
    CK(hipStreamSynchronize(s));                                                                                \
    float ms;                                                                                                   \
    CK(hipEventElapsedTime(&ms, a, b));                                                                         \
    const double us = ms * 1e3 / reps;                                                                          \
    std::printf("%5d (%d)%24s %5d  %-9s %6.1f %7.2f %7.2f\n", units, units == 174 ? 1 : units == 638 ? 4 : 8, "", W_, \
                SC_ ? "scattered" : "in a row", mb, us, mb / us);                                               \
  }
    TF_RUN(4, false) TF_RUN(4, true) TF_RUN(8, false) TF_RUN(8, true) TF_RUN(16, false) TF_RUN(16, true)
#undef TF_RUN
  }
  return 0;
}
