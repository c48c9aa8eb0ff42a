// Load-time repacking between the stored MLX layout and the kernels' layouts (both directions), one thread a word.
//
// Nibble order inside a packed word: slot p (bits 4p .. 4p+3) holds input 2 (p % 4) + p / 4 of the word's eight,
// so that (word >> 4 i) & 0x000F000F is the pair (input 2 i, input 2 i + 1) in the two bf16 halves of a dword.

#include "tf_common.h"

namespace tf {
namespace {

__device__ __forceinline__ uint32_t to_pairs(uint32_t w) {
  uint32_t r = 0;
#pragma unroll
  for (int p = 0; p < 8; ++p) r |= ((w >> (4 * (2 * (p & 3) + (p >> 2)))) & 15u) << (4 * p);
  return r;
}

__device__ __forceinline__ uint32_t from_pairs(uint32_t w) {
  uint32_t r = 0;
#pragma unroll
  for (int p = 0; p < 8; ++p) r |= ((w >> (4 * p)) & 15u) << (4 * (2 * (p & 3) + (p >> 2)));
  return r;
}

// out blocks [E, NB, KG, BW]; thread = one output word
__global__ void experts_pack_kernel(const uint32_t* __restrict__ words, const uint16_t* __restrict__ scales,
                                    const uint16_t* __restrict__ biases, uint32_t* __restrict__ out, int64_t total,
                                    int n, int k8, int kg, int gs) {
  const int bw = block_words(gs), cw = 32 * gs / 8, wpg = gs / 8;
  for (int64_t o = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; o < total; o += (int64_t)gridDim.x * blockDim.x) {
    const int q = (int)(o % bw);
    const int64_t blk = o / bw;
    const int g = (int)(blk % kg);
    const int64_t eb = blk / kg;                       // e * NB + nb
    const int nb = (int)(eb % (n / 32));
    const int64_t e = eb / (n / 32);
    if (q < cw) {
      const int i = q >> 7, c = (q >> 2) & 31, j = q & 3;
      out[o] = to_pairs(words[(e * n + nb * 32 + c) * k8 + g * wpg + i * 4 + j]);
    } else {
      const int c = q - cw;
      const int64_t at = (e * n + nb * 32 + c) * kg + g;
      out[o] = (uint32_t)scales[at] | ((uint32_t)biases[at] << 16);
    }
  }
}

// thread = one MLX word (and, for the first word of a group, the group's scale and bias)
__global__ void experts_unpack_kernel(const uint32_t* __restrict__ blocks, int64_t block_stride,
                                      uint32_t* __restrict__ words, uint16_t* __restrict__ scales,
                                      uint16_t* __restrict__ biases, int64_t total, int n, int k8, int kg, int gs) {
  const int cw = 32 * gs / 8, wpg = gs / 8;
  for (int64_t o = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; o < total; o += (int64_t)gridDim.x * blockDim.x) {
    const int kw = (int)(o % k8);
    const int64_t en = o / k8;                         // e * n + column
    const int col = (int)(en % n);
    const int64_t e = en / n;
    const int g = kw / wpg, r = kw % wpg, i = r >> 2, j = r & 3, nb = col >> 5, c = col & 31;
    const uint32_t* blk = blocks + ((e * (n / 32) + nb) * kg + g) * block_stride;
    words[o] = from_pairs(blk[i * 128 + c * 4 + j]);
    if (r == 0) {
      const uint32_t sb = blk[cw + c];
      scales[en * kg + g] = (uint16_t)(sb & 0xFFFFu);
      biases[en * kg + g] = (uint16_t)(sb >> 16);
    }
  }
}

// weight [npad/64, KG, gs/32, 64, 4]; thread = one output word; columns past n are zero
__global__ void qmm_pack_kernel(const uint32_t* __restrict__ words, uint32_t* __restrict__ weight, int64_t total, int n,
                                int k8, int kg, int gs) {
  const int ch = gs / 32;
  for (int64_t o = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; o < total; o += (int64_t)gridDim.x * blockDim.x) {
    const int j = (int)(o & 3), c = (int)((o >> 2) & 63);
    const int64_t rest = o >> 8;                       // (tile * kg + g) * ch + i
    const int i = (int)(rest % ch);
    const int g = (int)((rest / ch) % kg);
    const int64_t tile = rest / ch / kg;
    const int64_t col = tile * 64 + c;
    weight[o] = col < n ? to_pairs(words[col * k8 + g * (gs / 8) + i * 4 + j]) : 0u;
  }
}

__global__ void qmm_unpack_kernel(const uint32_t* __restrict__ weight, uint32_t* __restrict__ words, int64_t total,
                                  int k8, int kg, int gs) {
  const int ch = gs / 32, wpg = gs / 8;
  for (int64_t o = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; o < total; o += (int64_t)gridDim.x * blockDim.x) {
    const int kw = (int)(o % k8);
    const int64_t col = o / k8;
    const int g = kw / wpg, r = kw % wpg, i = r >> 2, j = r & 3;
    const int64_t tile = col >> 6;
    words[o] = from_pairs(weight[(((tile * kg + g) * ch + i) * 64 + (col & 63)) * 4 + j]);
  }
}

// dst[g, col] = src[col, g] for col < n, zero for n <= col < npad (and the inverse with `back`)
__global__ void sb_transpose_kernel(const uint16_t* __restrict__ src, uint16_t* __restrict__ dst, int n, int npad,
                                    int kg, int back) {
  const int64_t total = back ? (int64_t)n * kg : (int64_t)npad * kg;
  for (int64_t o = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; o < total; o += (int64_t)gridDim.x * blockDim.x) {
    if (back) {
      const int g = (int)(o % kg);
      const int64_t col = o / kg;
      dst[o] = src[(int64_t)g * npad + col];
    } else {
      const int64_t col = o % npad;
      const int g = (int)(o / npad);
      dst[o] = col < n ? src[col * kg + g] : (uint16_t)0;
    }
  }
}

inline unsigned blocks_for(int64_t total) {
  const int64_t b = (total + 255) / 256;
  return (unsigned)(b < 1 ? 1 : b > 65535 * 16 ? 65535 * 16 : b);
}

}  // namespace
}  // namespace tf

using namespace tf;

extern "C" int tf_experts_pack(const uint32_t* words, const uint16_t* scales, const uint16_t* biases, int e, int n,
                               int k, int gs, uint32_t* out, tf_stream_t stream) {
  clear_error();
  TF_REQUIRE(gs == 32 || gs == 64, "pack: groups of 32 or 64 inputs");
  TF_REQUIRE(words && scales && biases && out, "pack: null pointer argument");
  TF_REQUIRE(e >= 1 && n >= 32 && n % 32 == 0 && k >= gs && k % gs == 0,
             "pack: N must be a multiple of 32 and K of the group size");
  const int64_t total = (int64_t)e * (n / 32) * (k / gs) * block_words(gs);
  experts_pack_kernel<<<blocks_for(total), 256, 0, as_stream(stream)>>>(words, scales, biases, out, total, n, k / 8,
                                                                       k / gs, gs);
  TF_LAUNCH_OK("tf_experts_pack");
  return 0;
}

extern "C" int tf_experts_unpack(const uint32_t* blocks, int64_t block_stride, int e, int n, int k, int gs,
                                 uint32_t* words, uint16_t* scales, uint16_t* biases, tf_stream_t stream) {
  clear_error();
  TF_REQUIRE(gs == 32 || gs == 64, "unpack: groups of 32 or 64 inputs");
  TF_REQUIRE(blocks && words && scales && biases, "unpack: null pointer argument");
  TF_REQUIRE(e >= 1 && n >= 32 && n % 32 == 0 && k >= gs && k % gs == 0,
             "unpack: N must be a multiple of 32 and K of the group size");
  TF_REQUIRE(block_stride >= block_words(gs), "unpack: block stride smaller than a block");
  const int64_t total = (int64_t)e * n * (k / 8);
  experts_unpack_kernel<<<blocks_for(total), 256, 0, as_stream(stream)>>>(blocks, block_stride, words, scales, biases,
                                                                         total, n, k / 8, k / gs, gs);
  TF_LAUNCH_OK("tf_experts_unpack");
  return 0;
}

extern "C" int tf_qmm_pack(const uint32_t* words, const uint16_t* scales, const uint16_t* biases, int n, int k, int gs,
                           uint32_t* weight, uint16_t* scales_t, uint16_t* biases_t, tf_stream_t stream) {
  clear_error();
  TF_REQUIRE(gs == 32 || gs == 64, "pack: groups of 32 or 64 inputs");
  TF_REQUIRE(words && scales && biases && weight && scales_t && biases_t, "pack: null pointer argument");
  TF_REQUIRE(n >= 1 && k >= gs && k % gs == 0, "pack: K must be a multiple of the group size");
  const int npad = (n + 127) / 128 * 128, kg = k / gs;
  hipStream_t s = as_stream(stream);
  const int64_t total = (int64_t)npad * (k / 8);
  qmm_pack_kernel<<<blocks_for(total), 256, 0, s>>>(words, weight, total, n, k / 8, kg, gs);
  TF_LAUNCH_OK("tf_qmm_pack");
  const int64_t sbt = (int64_t)npad * kg;
  sb_transpose_kernel<<<blocks_for(sbt), 256, 0, s>>>(scales, scales_t, n, npad, kg, 0);
  sb_transpose_kernel<<<blocks_for(sbt), 256, 0, s>>>(biases, biases_t, n, npad, kg, 0);
  TF_LAUNCH_OK("tf_qmm_pack scales");
  return 0;
}

extern "C" int tf_qmm_unpack(const uint32_t* weight, const uint16_t* scales_t, const uint16_t* biases_t, int n, int k,
                             int gs, uint32_t* words, uint16_t* scales, uint16_t* biases, tf_stream_t stream) {
  clear_error();
  TF_REQUIRE(gs == 32 || gs == 64, "unpack: groups of 32 or 64 inputs");
  TF_REQUIRE(words && scales && biases && weight && scales_t && biases_t, "unpack: null pointer argument");
  TF_REQUIRE(n >= 1 && k >= gs && k % gs == 0, "unpack: K must be a multiple of the group size");
  const int npad = (n + 127) / 128 * 128, kg = k / gs;
  hipStream_t s = as_stream(stream);
  const int64_t total = (int64_t)n * (k / 8);
  qmm_unpack_kernel<<<blocks_for(total), 256, 0, s>>>(weight, words, total, k / 8, kg, gs);
  TF_LAUNCH_OK("tf_qmm_unpack");
  const int64_t sbt = (int64_t)n * kg;
  sb_transpose_kernel<<<blocks_for(sbt), 256, 0, s>>>(scales_t, scales, n, npad, kg, 1);
  sb_transpose_kernel<<<blocks_for(sbt), 256, 0, s>>>(biases_t, biases, n, npad, kg, 1);
  TF_LAUNCH_OK("tf_qmm_unpack scales");
  return 0;
}
