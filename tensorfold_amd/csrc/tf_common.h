// Shared by every translation unit of libtfmi: status/error plumbing, bf16 helpers, the 4-bit block geometry.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <cstdarg>
#include <cstdio>

#include "../../include/tfmi.h"

namespace tf {

// ---- status -------------------------------------------------------------------------------------------------------

void set_error(const char* fmt, ...);
void clear_error();

#define TF_REQUIRE(cond, ...)      \
  do {                             \
    if (!(cond)) {                 \
      ::tf::set_error(__VA_ARGS__); \
      return 1;                    \
    }                              \
  } while (0)

// after a launch: a sticky or launch-time error becomes a status
#define TF_LAUNCH_OK(what)                                                        \
  do {                                                                            \
    hipError_t e_ = hipGetLastError();                                            \
    if (e_ != hipSuccess) {                                                       \
      ::tf::set_error("%s: launch failed: %s", what, hipGetErrorString(e_));      \
      return 2;                                                                   \
    }                                                                             \
  } while (0)

inline hipStream_t as_stream(tf_stream_t s) { return reinterpret_cast<hipStream_t>(s); }
inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// ---- vector types ------------------------------------------------------------------------------------------------

typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4_t;
typedef __attribute__((ext_vector_type(16))) float f32x16_t;

// ---- bf16 ----------------------------------------------------------------------------------------------------------

__device__ __forceinline__ float bf16_lo(uint32_t v) { return __uint_as_float(v << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t v) { return __uint_as_float(v & 0xFFFF0000u); }
__device__ __forceinline__ float bf16_f32(uint16_t v) { return __uint_as_float(static_cast<uint32_t>(v) << 16); }

// round to nearest even (finite inputs; NaN stays NaN because the payload's top bit survives the add for quiet NaNs)
__device__ __forceinline__ uint32_t f32_bf16_bits(float f) {
  const uint32_t u = __float_as_uint(f);
  return (u + 0x7FFFu + ((u >> 16) & 1u)) >> 16;
}
__device__ __forceinline__ float round_bf16(float f) { return __uint_as_float(f32_bf16_bits(f) << 16); }
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
  return f32_bf16_bits(lo) | (f32_bf16_bits(hi) << 16);
}

// ---- epilogues (rounding points of the reference's experts.cuh:53-70) ---------------------------------------------

__device__ __forceinline__ float relu2(float a) {
  const float u = fmaxf(round_bf16(a), 0.f);
  return u * u;
}

__device__ __forceinline__ float swiglu(float g, float u, float limit) {
  float gv = round_bf16(g), uv = round_bf16(u);
  if (limit > 0.f) {
    gv = fminf(gv, limit);
    uv = fminf(fmaxf(uv, -limit), limit);
  }
  return round_bf16(gv / (1.f + __expf(-gv))) * uv;
}

// ---- issue priority by progress ------------------------------------------------------------------------------------
//
// A wave with `left` of its `n` loop trips to go takes priority 3 in the first quarter of them, down to 0 in the
// last: a wave that is behind issues first.  Left alone, the oldest wave of a SIMD issues first, the workgroups
// dispatched first finish microseconds before the others, and the launch ends on a few late ones that cannot fill
// the memory system by themselves.  (s_setprio takes an immediate, hence the switch.)
__device__ __forceinline__ void prio_by_progress(int left, int n) {
  const int left4 = 4 * left;
  switch (left4 > 3 * n ? 3 : left4 > 2 * n ? 2 : left4 > n ? 1 : 0) {
    case 3: __builtin_amdgcn_s_setprio(3); break;
    case 2: __builtin_amdgcn_s_setprio(2); break;
    case 1: __builtin_amdgcn_s_setprio(1); break;
    default: __builtin_amdgcn_s_setprio(0);
  }
}

// ---- timeline build -----------------------------------------------------------------------------------------------
//
// Compiled with -DTF_TIMELINE (libtfmi_timeline.so) the decode expert kernels note when thread 0 of each workgroup
// passes a few marks, on the 100 MHz clock every compute unit reads alike: 0 kernel entry, 1 the workgroup knows its
// item, 2 its first weights and inputs are requested, 3 wave 0 has streamed its share, 4 every wave has, 5 the unit
// has stored its output (and combined what it completed); a seventh row says which compute unit ran the workgroup,
// an eighth how many shader cycles (s_memtime) passed between marks 2 and 3, which against the marks' own 10 ns
// ticks is the clock the compute unit ran at.  The marks are kept in LDS and written out once, at mark
// 5 (a store to memory at each mark would put its round trip into the waits that follow it).  The ordinary build
// compiles the marks away.
#ifdef TF_TIMELINE
constexpr int TIMELINE_MARKS = 6, TIMELINE_ROWS = TIMELINE_MARKS + 2, TIMELINE_GROUPS = 16384;
static __device__ unsigned long long tf_timeline_marks[TIMELINE_ROWS][TIMELINE_GROUPS];
__device__ __forceinline__ unsigned long long* timeline_lds() {
  __shared__ unsigned long long t[TIMELINE_MARKS + 1];
  return t;
}
// `as` >= 0: the row of the table to write at the last mark (a workgroup that takes several units one after another
// marks each under the unit's number); otherwise the workgroup's own number
__device__ __forceinline__ void timeline_mark(int k, int as = -1) {
  if (threadIdx.x != 0) return;
  unsigned long long* t = timeline_lds();
  if (k == 0)
    for (int i = 1; i <= TIMELINE_MARKS; ++i) t[i] = 0;
  t[k] = wall_clock64();
  if (k == 2) t[TIMELINE_MARKS] = __builtin_readcyclecounter();
  if (k == 3) t[TIMELINE_MARKS] = __builtin_readcyclecounter() - t[TIMELINE_MARKS];
  const unsigned group = as >= 0 ? (unsigned)as : blockIdx.x + (blockIdx.y + blockIdx.z * gridDim.y) * gridDim.x;
  if (k == TIMELINE_MARKS - 1 && group < TIMELINE_GROUPS) {
    for (int i = 0; i < TIMELINE_MARKS; ++i) tf_timeline_marks[i][group] = t[i];
    // where it ran: the XCC id above the hardware id word (compute unit in bits 8-11, shader array 12, engine 13-15)
    tf_timeline_marks[TIMELINE_MARKS][group] =
        ((unsigned long long)__builtin_amdgcn_s_getreg((31 << 11) | 20) << 32) | __builtin_amdgcn_s_getreg((31 << 11) | 4);
    tf_timeline_marks[TIMELINE_MARKS + 1][group] = t[TIMELINE_MARKS];
  }
}
// The timeline build's two extra entry points of a source file that places marks: the marks of that file's last
// launches, [TIMELINE_ROWS][TIMELINE_GROUPS]: six rows of 64-bit ticks of 10 ns (0: never passed), then the row of
// hardware ids and the row of shader cycles between marks 2 and 3 (each source file has its own table).
#define TF_TIMELINE_EXPORT(NAME_)                                                                                   \
  extern "C" int tf_timeline_read_##NAME_(unsigned long long* host, int rows, int groups) {                         \
    ::tf::clear_error();                                                                                            \
    TF_REQUIRE(host && rows == ::tf::TIMELINE_ROWS && groups == ::tf::TIMELINE_GROUPS, "timeline: the table is %d x %d", \
               ::tf::TIMELINE_ROWS, ::tf::TIMELINE_GROUPS);                                                          \
    TF_REQUIRE(hipMemcpyFromSymbol(host, HIP_SYMBOL(::tf::tf_timeline_marks), sizeof(::tf::tf_timeline_marks)) ==    \
                   hipSuccess,                                                                                      \
               "timeline: the copy failed");                                                                        \
    return 0;                                                                                                       \
  }                                                                                                                 \
  extern "C" int tf_timeline_clear_##NAME_(void) {                                                                  \
    ::tf::clear_error();                                                                                            \
    static const unsigned long long zeros[::tf::TIMELINE_ROWS][::tf::TIMELINE_GROUPS] = {};                          \
    TF_REQUIRE(hipMemcpyToSymbol(HIP_SYMBOL(::tf::tf_timeline_marks), zeros, sizeof(zeros)) == hipSuccess,           \
               "timeline: the clear failed");                                                                       \
    return 0;                                                                                                       \
  }
#define TF_MARK(K_) timeline_mark(K_)
#define TF_MARK_AS(K_, AS_) timeline_mark(K_, AS_)
#else
#define TF_MARK(K_) \
  do {              \
  } while (0)
#define TF_MARK_AS(K_, AS_) \
  do {                      \
  } while (0)
#define TF_TIMELINE_EXPORT(NAME_)
#endif

// ---- 4-bit blocks -------------------------------------------------------------------------------------------------

constexpr uint32_t NIB_MASK = 0x000F000Fu;
constexpr uint32_t BF16_ONES = 0x3F803F80u;  // the bf16 pair (1, 1)
constexpr uint32_t BF16_128 = 0x43004300u;   // the bf16 pair (128, 128): OR-ing a nibble into the mantissa gives 128 + q

// int32 words of an experts block: 32 columns x gs inputs of codes, then 32 (scale | bias << 16) words
__host__ __device__ constexpr int block_words(int gs) { return 32 * gs / 8 + 32; }

}  // namespace tf
