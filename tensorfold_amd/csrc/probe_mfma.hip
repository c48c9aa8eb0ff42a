// Issue rates of the matrix instructions a prompt-form kernel could be built on, measured on the GPU it runs on:
// v_mfma_f32_16x16x32_f16 (what the prompt kernels use), v_mfma_f32_32x32x16_f16, v_mfma_f32_16x16x32_fp8_fp8 and the
// block-scaled v_mfma_scale_f32_16x16x128_f8f6f4, bare (a loop of nothing else, independent accumulators) and with
// the work the affine format needs between groups on 8-bit operands: a partial sum zeroed, accumulated over one
// group of 32 or 64 inputs, then acc = fma(P, scale, acc) (the arithmetic of the reference's
// cuda/kernels/qmm_prefill8.cu:1-2).  A stand-alone program: `python bench_configs.py mfma` builds nothing and runs
// the binary that tensorfold_amd/build.py compiled beside the library.
#include <hip/hip_runtime.h>
#include <cstdio>
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(8))) int i32x8;

template <int WHICH, int T>
__global__ void __launch_bounds__(256) probe(float* out, int iters) {
  const int lane = threadIdx.x & 63;
  f16x8 a, b;
  for (int i = 0; i < 8; ++i) { a[i] = (_Float16)(lane * 0.01f + i); b[i] = (_Float16)(i * 0.5f - lane * 0.02f); }
  long a8 = 0x3838383838383838L + lane, b8 = 0x4040404040404040L - lane;
  float r = 0;
  if constexpr (WHICH == 0 || WHICH == 2) {
    f32x4 acc[T];
    for (int t = 0; t < T; ++t) acc[t] = (f32x4){0, 0, 0, 0};
    for (int k = 0; k < iters; ++k)
#pragma unroll
      for (int t = 0; t < T; ++t) {
        if (WHICH == 0) asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+v"(acc[t]) : "v"(a), "v"(b));
        else asm volatile("v_mfma_f32_16x16x32_fp8_fp8 %0, %1, %2, %0" : "+v"(acc[t]) : "v"(a8), "v"(b8));
      }
    for (int t = 0; t < T; ++t) r += acc[t][0] + acc[t][3];
  } else {
    f32x16 acc[T];
    for (int t = 0; t < T; ++t) for (int j = 0; j < 16; ++j) acc[t][j] = 0;
    for (int k = 0; k < iters; ++k)
#pragma unroll
      for (int t = 0; t < T; ++t) asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(acc[t]) : "v"(a), "v"(b));
    for (int t = 0; t < T; ++t) r += acc[t][0] + acc[t][9];
  }
  out[blockIdx.x * 256 + threadIdx.x] = r;
}

// the affine format's prompt arithmetic on 8-bit operands: P zeroed, accumulated over one group of G inputs, then
// acc = fma(P, s, acc): what qmm_prefill8 does between groups (4 VALU a tile a group, plus the zeroing)
template <int WHICH, int G>
__global__ void __launch_bounds__(256) grouped(float* out, int iters, float s) {
  constexpr int T = 8, IPG = G / 32;
  const int lane = threadIdx.x & 63;
  f16x8 a, b;
  for (int i = 0; i < 8; ++i) { a[i] = (_Float16)(lane * 0.01f + i); b[i] = (_Float16)(i * 0.5f - lane * 0.02f); }
  long a8 = 0x3838383838383838L + lane, b8 = 0x4040404040404040L - lane;
  f32x4 acc[T], p[T];
  for (int t = 0; t < T; ++t) acc[t] = (f32x4){0, 0, 0, 0};
  for (int k = 0; k < iters; k += IPG) {
#pragma unroll
    for (int t = 0; t < T; ++t) p[t] = (f32x4){0, 0, 0, 0};
#pragma unroll
    for (int i = 0; i < IPG; ++i)
#pragma unroll
      for (int t = 0; t < T; ++t) {
        if (WHICH == 0) asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+v"(p[t]) : "v"(a), "v"(b));
        else asm volatile("v_mfma_f32_16x16x32_fp8_fp8 %0, %1, %2, %0" : "+v"(p[t]) : "v"(a8), "v"(b8));
      }
    asm volatile("s_nop 15\n s_nop 15" ::: "memory");        // the last MFMA's result must land before a VALU reads it
#pragma unroll
    for (int t = 0; t < T; ++t)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[t][j] = fmaf(p[t][j], s, acc[t][j]);
  }
  float r = 0;
  for (int t = 0; t < T; ++t) r += acc[t][0] + acc[t][3];
  out[blockIdx.x * 256 + threadIdx.x] = r;
}

template <int WHICH, int G>
void run_grouped(const char* name, float* out, int blocks) {
  const int iters = 8192;
  hipEvent_t e0, e1; (void)hipEventCreate(&e0); (void)hipEventCreate(&e1);
  float best = 1e9f, ms;
  for (int rep = 0; rep < 8; ++rep) {
    (void)hipEventRecord(e0);
    grouped<WHICH, G><<<blocks, 256>>>(out, iters, 1.0009765625f);
    (void)hipEventRecord(e1); (void)hipEventSynchronize(e1);
    (void)hipEventElapsedTime(&ms, e0, e1);
    if (ms < best) best = ms;
  }
  const double instr = (double)blocks * 4 * 8 * iters;
  printf("%-26s group %3d %d waves/SIMD %8.3f ms %7.1f TFLOP/s %5.1f cycles an MFMA a SIMD at 2.4 GHz\n", name, G, blocks * 4 / 1024,
         best, instr * 16384.0 / best * 1e-9, best * 1e-3 * 2.4e9 / (instr / 1024));
}

__global__ void __launch_bounds__(256) probe_f8f6f4(float* out, int iters) {
  const int lane = threadIdx.x & 63;
  i32x8 a, b;
  for (int i = 0; i < 8; ++i) { a[i] = 0x38383838 + lane + i; b[i] = 0x40404040 - lane - i; }
  f32x4 acc[4];
  for (int t = 0; t < 4; ++t) acc[t] = (f32x4){0, 0, 0, 0};
  for (int k = 0; k < iters; ++k)
#pragma unroll
    for (int t = 0; t < 4; ++t)
      acc[t] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, acc[t], 0, 0, 0, 0x7F7F7F7F, 0, 0x7F7F7F7F);
  float r = 0;
  for (int t = 0; t < 4; ++t) r += acc[t][0] + acc[t][3];
  out[blockIdx.x * 256 + threadIdx.x] = r;
}

void run_f8f6f4(float* out, int blocks) {
  const int iters = 8192;
  hipEvent_t e0, e1; (void)hipEventCreate(&e0); (void)hipEventCreate(&e1);
  float best = 1e9f, ms;
  for (int rep = 0; rep < 8; ++rep) {
    (void)hipEventRecord(e0);
    probe_f8f6f4<<<blocks, 256>>>(out, iters);
    (void)hipEventRecord(e1); (void)hipEventSynchronize(e1);
    (void)hipEventElapsedTime(&ms, e0, e1);
    if (ms < best) best = ms;
  }
  const double instr = (double)blocks * 4 * 4 * iters;
  printf("%-26s T=4 %d waves/SIMD %8.3f ms %7.1f TFLOP/s %5.1f cycles an MFMA a SIMD at 2.4 GHz\n", "f8f6f4 16x16x128 (fp8)", blocks * 4 / 1024,
         best, instr * 65536.0 / best * 1e-9, best * 1e-3 * 2.4e9 / (instr / 1024));
}

template <int WHICH, int T>
void run(const char* name, float* out, int blocks) {
  const int iters = 8192;
  hipEvent_t e0, e1; (void)hipEventCreate(&e0); (void)hipEventCreate(&e1);
  float best = 1e9f, ms;
  for (int rep = 0; rep < 8; ++rep) {
    (void)hipEventRecord(e0);
    probe<WHICH, T><<<blocks, 256>>>(out, iters);
    (void)hipEventRecord(e1); (void)hipEventSynchronize(e1);
    (void)hipEventElapsedTime(&ms, e0, e1);
    if (ms < best) best = ms;
  }
  const double instr = (double)blocks * 4 * T * iters;
  const double flop = instr * (WHICH == 1 ? 2.0 * 32 * 32 * 16 : 2.0 * 16 * 16 * 32);
  printf("%-26s T=%d %d waves/SIMD %8.3f ms %7.1f TFLOP/s %5.1f cycles an MFMA a SIMD at 2.4 GHz\n", name, T, blocks * 4 / 1024, best,
         flop / best * 1e-9, best * 1e-3 * 2.4e9 / (instr / 1024));
}

int main() {
  float* out; (void)hipMalloc(&out, 4 * 256 * 4096);
  run<0, 8>("f16 16x16x32", out, 256);
  run<0, 8>("f16 16x16x32", out, 512);
  run<0, 8>("f16 16x16x32", out, 1024);
  run<0, 4>("f16 16x16x32", out, 512);
  run<0, 2>("f16 16x16x32", out, 512);
  run<1, 4>("f16 32x32x16", out, 256);
  run<1, 4>("f16 32x32x16", out, 512);
  run<1, 2>("f16 32x32x16", out, 512);
  run<2, 8>("fp8 16x16x32", out, 512);
  run<2, 8>("fp8 16x16x32", out, 1024);
  run_f8f6f4(out, 512);
  run_f8f6f4(out, 1024);
  run_grouped<0, 32>("f16 16x16x32 + fma/group", out, 512);
  run_grouped<0, 64>("f16 16x16x32 + fma/group", out, 512);
  run_grouped<1, 32>("fp8 16x16x32 + fma/group", out, 512);
  run_grouped<1, 64>("fp8 16x16x32 + fma/group", out, 512);
  run_grouped<1, 32>("fp8 16x16x32 + fma/group", out, 1024);
  run_grouped<1, 64>("fp8 16x16x32 + fma/group", out, 1024);
  return 0;
}
