/* libtfmi: MI355X (gfx950) kernels for TensorFold's quantized routed-expert matmul path, C ABI.
 *
 * Every entry point takes raw device pointers, sizes and a hipStream_t (passed as void*), launches on that stream
 * without synchronising or allocating, and returns 0 on success or a non-zero status; tf_last_error() then holds a
 * sentence naming the offending argument (thread-local).  All buffers are caller-owned.  Launches are safe to
 * capture in a hipGraph: no host reads of device data, grid sizes come from host-side upper bounds.
 *
 * Each declaration cites the binding of the reference's CUDA extension it replaces (paths relative to
 * src/tensorfold/cuda/ in the reference tree).
 *
 * Packed layouts (ours; callers only rely on the outer dimensions):
 *   experts table  int32 [E, N/32, K/gs, M, 32*gs/8 + 32]   M = 2 (gate, up) or 1
 *       block (32 columns x one group): gs/32 chunks of [32 columns][4 words], then [32 columns] (scale | bias << 16)
 *       word j of a column's chunk holds inputs 8 j .. 8 j + 7; nibble slot p (bits 4p..4p+3) holds input
 *       2 (p % 4) + p / 4, so (word >> 4 i) & 0x000F000F is the pair (input 2 i, input 2 i + 1)
 *   lane weight Q4 int32 [npad/64, K/gs, gs/32, 64, 4]  (same chunk and nibble order, 64 columns a tile),
 *       scales and biases bf16 [K/gs, npad], npad = n rounded up to 128
 */
#ifndef TFMI_H
#define TFMI_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* tf_stream_t; /* hipStream_t */

/* dtype codes for EXL3 inputs and outputs (exl3/linear.cu:16 `enum DType`) */
enum { TF_F16 = 0, TF_BF16 = 1, TF_F32 = 2 };

/* ---- library ------------------------------------------------------------------------------------------------- */

/* The message of the last failing call on this thread ("" if none). */
const char* tf_last_error(void);
/* ABI version of this header: 3 (tf_moe_decode_sliced added; tf_experts_prefill's `counts` holds four int32). */
int tf_version(void);
/* Digest of the sources and compiler flags the library was built from (16 hex digits), "unknown" when the build gave
 * none.  The Python loader compares it with the sources beside it before it loads the file. */
const char* tf_build_id(void);
/* 0 when the current HIP device is gfx950; otherwise non-zero with a message naming the device.
 * Replaces build.py:20-32 `arch_flags` (refusal of a GPU the kernels were not built for). */
int tf_check_device(void);

/* ---- affine 4-bit lane matmul (kernels/qmm.cpp:151-157, module tensorfold_qmm_v5) --------------------------------- */

/* MLX (n, k/8) words and (n, k/gs) bf16 scales/biases -> Q4 weight, (k/gs, npad) scales and biases.
 * Replaces kernels/qmm.py:72-99 `pack` (torch ops in the reference, one kernel here). */
int tf_qmm_pack(const uint32_t* words, const uint16_t* scales, const uint16_t* biases, int n, int k, int gs,
                uint32_t* weight, uint16_t* scales_t, uint16_t* biases_t, tf_stream_t stream);
/* The inverse: kernels/qmm.py:102-119 `unpack`. */
int tf_qmm_unpack(const uint32_t* weight, const uint16_t* scales_t, const uint16_t* biases_t, int n, int k, int gs,
                  uint32_t* words, uint16_t* scales, uint16_t* biases, tf_stream_t stream);
/* xs[m, g] = fp32 sum of x[m, g*gs .. (g+1)*gs).  Replaces kernels/qmm.py:139-154 `group_sums` (Triton). */
int tf_group_sums(const uint16_t* x, int64_t ldx, int m, int k, int gs, float* xs, tf_stream_t stream);
/* Decode-form matmul: per group in order acc = fma(xs, b, fma(P, s, acc)), P = sum x*q with exact q; K in `sk`
 * slices summed in slice order; one rounding to bf16 (or fp32 with f32).  `part` fp32 [sk, m, n] is required when
 * sk > 1 (with reduce == 0 the slices are left there unadded; with few rows and reduce != 0 the slices are added
 * inside the one launch, in the same order, and `part` goes unused).  sb_stride = elements between scale rows
 * (>= npad).  `counters` (may be NULL): n_counters arrival counters of the weight, TF_QMM_COUNTER_STRIDE ints apart,
 * zero on entry and left zero; with one for every column tile of 64, the slices of up to eight rows are added up in the
 * matmul's own launch by the last workgroup of a tile to finish (same order, same bits);
 * calls on one weight's counters must not overlap.  Replaces kernels/qmm.cpp:18-48 `qmm`. */
#define TF_QMM_COUNTER_STRIDE 16
int tf_qmm(const uint16_t* x, int64_t ldx, const float* xs, const uint32_t* weight, const uint16_t* scales,
           const uint16_t* biases, int64_t sb_stride, void* out, float* part, int32_t* counters, int n_counters, int m,
           int n, int k, int sk, int gs, int bm, int f32, int reduce, tf_stream_t stream);
/* tf_qmm (reduce != 0) for callers that cannot allocate or pass a workspace: code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc.  The K slices that tf_qmm keeps in `part` live in a fixed array
 * inside the library's device image (TF_QMM_STATIC_FLOATS fp32 = 16 MiB, held by every GPU the library runs on
 * until the process ends); sk * m * n beyond that is refused with a message.  Nothing is allocated or freed by the
 * call.  Same kernels and bits as tf_qmm.  Every call on a GPU shares that GPU's array: calls that overlap on one
 * GPU (two streams, two threads) race; calls on one stream are ordered.  Nothing in the array needs to start at
 * zero (each slice is written in full before it is read).  The arrival counters that let up to eight rows finish in
 * one launch live in the device image too (TF_QMM_STATIC_COUNTERS of them, 256 KiB; zero when the image is loaded,
 * put back to zero by every launch; a weight of more column tiles of 64 than that takes tf_qmm's counter-less
 * forms).  No counterpart in the reference, whose `qmm` allocates `part` itself when none is given
 * (kernels/qmm.cpp:40-45). */
#define TF_QMM_STATIC_FLOATS (4u << 20)
#define TF_QMM_STATIC_COUNTERS 4096
int tf_qmm_static(const uint16_t* x, int64_t ldx, const float* xs, const uint32_t* weight, const uint16_t* scales,
                  const uint16_t* biases, int64_t sb_stride, void* out, int m, int n, int k, int sk, int gs, int bm,
                  int f32, tf_stream_t stream);
/* `count` (1 to 4) weights against one x in one launch (plus one reduce launch when any K is split and the rows are
 * many): the bits of tf_qmm on each.  The arrays are host arrays of `count` entries, read during the call: packed weights, transposed
 * scales and biases with their row strides, outputs, parts (fp32 [sks[i], m, ns[i]], may be NULL where sks[i] == 1),
 * column counts and slice counts; `counters` (may be NULL) the weights' arrival counters with their counts, as in
 * tf_qmm: with them up to eight rows take one launch in which every weight's slices are added up by the last
 * workgroup of a tile.  Replaces kernels/qmm.cpp:51-80 `qmm_group`. */
int tf_qmm_group(const uint16_t* x, int64_t ldx, const float* xs, int count, const uint32_t* const* weights,
                 const uint16_t* const* scales, const uint16_t* const* biases, const int64_t* sb_strides,
                 void* const* outs, float* const* parts, int32_t* const* counters, const int* n_counters, const int* ns,
                 const int* sks, int m, int k, int gs, int bm, int f32, tf_stream_t stream);
/* The arithmetic of the prompt-form (MFMA) matmuls.
 *   TF_ARITH_F16: operands in fp16 - each weight rounded once as fp16(256 w), activations converted to fp16 (exact for a
 *     bf16 value between 2^-14 and 65504 in magnitude; larger ones are clamped to +-65504, smaller ones keep 2^-24
 *     absolute).  Valid when every |scale| and |bias| of the table is below 255.9 (256 x must stay finite in fp16)
 *     and the activations stay within +-65504.  An eighth of the reference's weight rounding error: the form that
 *     holds 2e-3 relative L2 against dequant-then-matmul in fp32, and the fast one.
 *   TF_ARITH_BF16: the reference's own arithmetic - w = bf16(fma(q, s, b)) (round to nearest even), bf16 activations
 *     untouched, bf16 MFMA (kernels/qmm_prefill.cu:116-117, experts_prefill.cu:130-131).  bf16's range on both
 *     operands; the same kernels (twice the vector instructions a weight: each is an fp32 fma rounded to bf16).
 * The Python wrappers choose TF_ARITH_BF16 by themselves for a table whose scales or biases do not fit the fp16 form. */
enum { TF_ARITH_F16 = 0, TF_ARITH_BF16 = 1 };

/* Prompt-form matmul on MFMA: each weight rounded once (see TF_ARITH_*), one fp32 chain over K.
 * tile: 0 = chosen from the row count (what kernels/qmm.py:202-205 `prompt_tile` stands for); 1, 4, 8 = the four-wave
 * kernel on 16, 64 or 128 rows a workgroup; 9 = the eight-wave kernel (128 rows x 512 columns; K in whole steps of
 * 64 only).  A row's bits are the same whatever the tile.
 * Replaces kernels/qmm.cpp:83-102 `qmm_prefill`. */
int tf_qmm_prefill(const uint16_t* x, int64_t ldx, const uint32_t* weight, const uint16_t* scales,
                   const uint16_t* biases, void* out, int m, int n, int k, int gs, int f32, int tile, int arith,
                   tf_stream_t stream);

/* The FP8 prompt path.  tf_quantize_rows: a row's scale a = max|x| / 448 (1 for a row of zeros), x8 = OCP e4m3 of
 * x / a (round to nearest even), xs[g] = bf16(sum of group g's inputs / a); x8 uint8 [m, k] with every octet of
 * inputs stored in the matrix operand's order (0, 4, 1, 5, 2, 6, 3, 7), xs bf16 [m, k / gs], a fp32 [m]; k a multiple
 * of gs and of 32.  Replaces kernels/qmm.py:222-255 `quantize_rows` (Triton).
 * tf_qmm_prefill8: out = (sum over groups, in order, of fma(P, scale, .) with P = the group's sum of x8 * code, exact
 * e4m3 operands; + xs . bias over the groups) * a, on tf_quantize_rows' output and a packed weight; out fp32 (f32) or
 * bf16 [m, n]; k in whole steps of 64; a row's bits depend on that row alone; `tile` (0-11) is accepted and changes
 * nothing.  Replaces kernels/qmm.cpp:151-157 `qmm_prefill8` (kernels/qmm_prefill8.cu). */
int tf_quantize_rows(const uint16_t* x, int64_t ldx, int m, int k, int gs, uint8_t* x8, uint16_t* xs, float* a,
                     tf_stream_t stream);
int tf_qmm_prefill8(const uint8_t* x8, const uint16_t* xs, const float* a, const uint32_t* weight,
                    const uint16_t* scales, const uint16_t* biases, void* out, int m, int n, int k, int gs, int f32,
                    int tile, tf_stream_t stream);

/* ---- routed experts (experts.cpp:77-82, module tensorfold_experts_v7) ---------------------------------------------- */

/* MLX words [E, N, K/8], scales/biases [E, N, K/gs] -> blocks [E, N/32, K/gs, 32*gs/8 + 32].
 * Replaces experts.cpp:57-75 `pack`. */
int tf_experts_pack(const uint32_t* words, const uint16_t* scales, const uint16_t* biases, int e, int n, int k,
                    int gs, uint32_t* out, tf_stream_t stream);
/* The inverse (experts.py:43-59 `unpack`, torch ops in the reference).  `blocks` may be one matrix of a stacked
 * table: block_stride = int32 elements between consecutive (column block, group) blocks. */
int tf_experts_unpack(const uint32_t* blocks, int64_t block_stride, int e, int n, int k, int gs, uint32_t* words,
                      uint16_t* scales, uint16_t* biases, tf_stream_t stream);
/* Stable grouping of pairs p = row*slots + slot by expert: members [pairs], items [(expert, first, count<=tile)],
 * counts = {items, distinct experts} (four int32 where the plan goes to tf_experts_prefill, see there).  rank [pairs]
 * and hist [ceil(pairs/1024) * experts] are scratch, used when pairs > 1024.  tile is 16 (decode), 64 or 128
 * (prefill).  Replaces experts.cpp:33-41 `plan`. */
int tf_experts_plan(const int32_t* picks, int64_t pairs, int experts, int tile, int32_t* members, int32_t* items,
                    int32_t* counts, int32_t* rank, int32_t* hist, tf_stream_t stream);
/* Decode form.  epi 0: fp32 out; 1: bf16 relu(bf16 a)^2; 2: bf16 SwiGLU(matrix 0, matrix 1) with clip `limit`.
 * Pair p reads x row p / slots when slots > 0, row p when slots == 0.  max_units = max items * nb bounds the grid;
 * the live item count is read on the device.  The group sums of the inputs that the affine form needs are taken
 * by each wave from the inputs it streams (no separate pass, no buffer).  Replaces experts.cpp:43-48 `run`. */
int tf_experts_run(int gs, int epi, const uint16_t* x, int64_t x_stride, int slots, const uint32_t* w, int kg, int nb,
                   const int32_t* items, const int32_t* counts, const int32_t* members, void* out, int n, float limit,
                   int64_t max_units, tf_stream_t stream);
/* Item descriptors, written by tf_moe_route_decode and tf_moe_route_up for the decode expert kernels: int32 rows of
 * TF_DESC_INTS; row 0 holds the number of descriptors, row 1 + i = {expert, count, first member, 0, pairs[..]}: the plan
 * cut into items of at most TF_DESC_TILE pairs, every full item first (expert order), then the experts' short last
 * items (expert order).  A buffer for P pairs over E experts needs
 * 1 + min(P, min(P, E) + P / TF_DESC_TILE) rows (no item is empty); that bound is the max_items of the calls that
 * read descriptors. */
#define TF_DESC_INTS 8
#define TF_DESC_TILE 2
/* ints between two descriptors' arrival counters in tf_moe_decode_experts' `done` (each alone in 256 bytes) */
#define TF_DONE_STRIDE 64
/* ints between two cells' arrival counters in `arrive` when rows <= 64 (each alone in 64 bytes); 1 past 64 rows */
#define TF_ARRIVE_STRIDE 16

/* tf_experts_run with the items given as descriptors; counts is not read (kept for symmetry).
 * Same bits as tf_experts_run on the same plan.  Same reference counterpart (experts.cpp:43-48 `run`); the
 * descriptor form has none. */
int tf_experts_run_desc(int gs, int epi, const uint16_t* x, int64_t x_stride, int slots, const uint32_t* w, int kg,
                        int nb, const int32_t* desc, const int32_t* counts, void* out, int n, float limit,
                        int64_t max_items, tf_stream_t stream);
/* Prompt form on MFMA, each weight rounded once as in tf_qmm_prefill (arith: TF_ARITH_*); epi 3: bf16 out; epi 4: fp16
 * out, values beyond fp16's range stored as +-65504.  `tile` is the plan's item size (16, 64 or 128).
 * `counts` holds FOUR int32 here: {items, distinct experts} as tf_experts_plan left them, then a ticket word and a
 * spare, both zero when the buffer is made.  Large plans run on one workgroup a compute unit, and the workgroups
 * draw their work from the ticket word; the launch leaves it at zero again, so nothing has to clear it between
 * launches, and launches that share a `counts` buffer must not overlap (one stream, or one after the other).
 * Replaces experts.cpp:50-55 `prefill`. */
int tf_experts_prefill(int gs, int epi, const uint16_t* x, int64_t x_stride, int slots, const uint32_t* w, int kg,
                       int nb, const int32_t* items, int32_t* counts, const int32_t* members, void* out, int n,
                       float limit, int64_t max_items, int tile, int arith, tf_stream_t stream);

/* ---- MoE glue (moe.py:23-151; Triton kernels in the reference) ------------------------------------------------------ */

/* logits[m, e] = fp32 x[m] . rows[e]  (bf16 inputs).  Replaces moe.py:23-55 `_router` / `router`. */
int tf_moe_router(const uint16_t* x, int64_t ldx, const uint16_t* rows, float* logits, int m, int d, int ne,
                  tf_stream_t stream);
/* Per row: top_k of logits[r, 0..experts) (largest first, lower id on ties), weights bf16(exp(l_k - l_0)/sum) as
 * fp32; with shared != 0 slot top_k is expert id `experts` weighted bf16(sigmoid(bf16(logits[r, experts]))).
 * pick int32 and wts fp32 are [rows, top_k + (shared ? 1 : 0)].  Replaces moe.py:58-108 `_topk_rows` / `select_rows`. */
int tf_moe_topk(const float* logits, int64_t ldl, int rows, int experts, int top_k, int shared, int32_t* pick,
                float* wts, tf_stream_t stream);
/* out[r] = bf16(sum_k wts[r, k] * y[r, k]) in slot order, fp32; y is fp32 (y_bf16 == 0), bf16 (1) or fp16 (2).
 * Replaces moe.py:131-151 `_combine` / `combine`. */
int tf_moe_combine(const void* y, int y_bf16, const float* wts, uint16_t* out, int rows, int slots, int d,
                   tf_stream_t stream);

/* The producers of a 4-bit matmul's input in one launch, a row's bits depending on that row alone:
 *   hn = x                                   (delta_kind 0; h is not written and may be NULL)
 *      = bf16(x + delta)                     (1: delta bf16 [rows, d])
 *      = bf16(x + bf16(routed + shared))     (2, 3: delta = pair outputs [rows * slots, d], fp32 or bf16;
 *                                             routed = sum over slots < `routed` of wts[r, k] * y[r, k], shared = sum
 *                                             of the other slots' y[r, k], fp32 in slot order)
 *   y  = bf16(hn / sqrt(mean(hn^2) + eps) * w),  xs[r, g] = fp32 sum of y over group g of `gs` columns.
 * x, w, h, y bf16; xs fp32 [rows, d / gs]; d <= 16384, whole groups of gs = 32, 64 or 128.
 * Replaces families/qwen3_5/cuda/glue.py:10-41 `add_rmsnorm` and families/nemotron_h/cuda/glue.py:103-141
 * `add_moe_norm`. */
int tf_add_norm(const uint16_t* x, const void* delta, int delta_kind, const float* wts, int slots, int routed,
                const uint16_t* w, float eps, uint16_t* h, uint16_t* y, float* xs, int rows, int d, int gs,
                tf_stream_t stream);

/* Routing and the up projection of the decode layer in ONE launch, for rows * (top_k + shared) <= 1024: workgroup 0
 * writes what tf_moe_topk and tf_experts_plan (tile 16) would (pick, wts, members, items, counts) plus the item
 * descriptors that tf_experts_run_desc reads; every other workgroup finds its own item from the
 * logits (with 2 to 64 rows a workgroup a pair: its own row's selection up to its slot, then a rank test of that
 * expert on the other rows) and runs the up unit of tf_experts_run (epilogue relu^2, or SwiGLU when swiglu != 0): act
 * bf16 [pairs, ni]; it also zeroes `zero` (n_zero ints: the next launch's counters).  Same
 * bits as the separate calls.  logits may be NULL: pick and wts are then inputs (tf_moe_topk ran before, the better
 * order past about 2,048 logits, where reading the rows in every workgroup costs more than a launch) and every
 * workgroup finds its item from the picks.  No counterpart in the reference (moe.py:88-128 issues them one by one). */
int tf_moe_route_up(const float* logits, int64_t ldl, int rows, int experts, int top_k, int shared, int gs, int swiglu,
                    const uint16_t* x, int64_t x_stride, const uint32_t* up, int d, int ni, int32_t* pick, float* wts,
                    int32_t* members, int32_t* items, int32_t* counts, int32_t* desc, uint16_t* act, float limit,
                    int max_items, int32_t* zero, int n_zero, tf_stream_t stream);
/* The down projection from item descriptors with the weighted combine folded in: y fp32 [pairs, d] as
 * tf_experts_run_desc (epilogue 0) writes it, and out bf16 [rows, d] with the bits of tf_moe_combine, written by
 * whichever workgroup completes a (token, 64 columns) cell.  `arrive` int32 [rows * ceil(d / 64) * s], s =
 * TF_ARRIVE_STRIDE with rows <= 64 and 1 past that, must be zero on
 * entry (tf_moe_route_up and tf_moe_route_decode clear a `zero` range for this); the workgroup that completes a cell
 * sets its counter back to zero, so a cell every slot of which held a valid expert is left at zero.  Fuses
 * experts.cpp:43-48 `run` and moe.py:131-151 `combine`. */
int tf_moe_down_combine(int gs, const uint16_t* act, int rows, int slots, const uint32_t* down, int d, int ni,
                        const int32_t* desc, const float* wts, float* y, uint16_t* out, int32_t* arrive,
                        int max_items, tf_stream_t stream);
/* The whole decode layer in ONE launch, cut along the intermediate width: tf_moe_route_up followed by
 * tf_moe_down_combine, same outputs (pick, wts, members, items, counts, desc, act, y, out) and the same bits.  A
 * workgroup takes (item of one or two pairs, 64 columns of ni): the up unit, then the part of the down projection those
 * 64 activations feed, for all d columns; it leaves each group's term fp32 in `part` [pairs, d / 64, ni / gs, 64], and
 * the workgroup that brings a (pair, 64 columns of d) cell its last group adds the terms in the down launch's order,
 * the one that then completes a (token, 64 columns) cell adds the slots (nobody waits).  d and ni multiples of 64;
 * `arrive` int32 [(pairs + rows) * (d / 64) * TF_ARRIVE_STRIDE], zero on entry and left at zero.  With logits the
 * weights of a combine are taken from the token's logits again; with logits NULL pick and wts are inputs.  No
 * counterpart in the reference, which splits a layer's intermediate width only across GPUs
 * (families/nemotron_h/cuda/tp.py:38-51). */
int tf_moe_decode_sliced(const float* logits, int64_t ldl, int rows, int experts, int top_k, int shared, int gs,
                         int swiglu, const uint16_t* x, int64_t x_stride, const uint32_t* up, const uint32_t* down,
                         int d, int ni, int32_t* pick, float* wts, int32_t* members, int32_t* items, int32_t* counts,
                         int32_t* desc, uint16_t* act, float* y, uint16_t* out, float* part, int32_t* arrive,
                         float limit, int max_items, tf_stream_t stream);
/* The decode layer's routing in one launch (two past 16 rows: the top-k then runs a workgroup a row first), for
 * rows * (top_k + shared) <= 1024: tf_moe_topk and tf_experts_plan (tile 16), plus the item descriptors and the
 * zeroing of `zero` (n_zero ints: the counters of tf_moe_down_combine or tf_moe_decode_experts).  No counterpart in
 * the reference, which launches `_topk_rows` and `plan` separately (moe.py:103-116). */
int tf_moe_route_decode(const float* logits, int64_t ldl, int rows, int experts, int top_k, int shared, int32_t* pick,
                        float* wts, int32_t* members, int32_t* items, int32_t* counts, int32_t* desc, int32_t* zero,
                        int n_zero, tf_stream_t stream);
/* The decode layer's experts in one launch: up (+ relu^2 or SwiGLU), down and the weighted combine, with the bits
 * of tf_experts_run, tf_experts_run and tf_moe_combine run in turn.  desc, counts, wts as left by
 * tf_moe_route_decode; scratch act bf16 [pairs, ni], y fp32 [pairs, d]; counters done
 * [max_items * 64] (one a descriptor, each alone in 256 bytes: TF_DONE_STRIDE ints apart) and arrive [rows * d/64 * s] (s as in tf_moe_down_combine) zero on entry; status[0] is set to 1 if a bounded wait ran out (the output
 * is then invalid).  d and ni multiples of 64.  Fuses experts.cpp:43-48 `run` (twice) and moe.py:131-151 `combine`. */
int tf_moe_decode_experts(int gs, int swiglu, const uint16_t* x, int64_t x_stride, int rows, int slots,
                          const uint32_t* up, const uint32_t* down, int d, int ni, const int32_t* desc,
                          const int32_t* counts, const float* wts, uint16_t* act, float* y, uint16_t* out,
                          int32_t* done, int32_t* arrive, int32_t* status, float limit, int max_items,
                          tf_stream_t stream);

#define TF_EXL3_COUNTER_STRIDE 16

/* ---- EXL3 linear (exl3/linear.cpp:70-74, module tensorfold_exl3_linear_v3) ---------------------------------------- */

/* xh[m, k] fp16 = fp16(((x * suh) @ H) / sqrt(128)) per block of 128; x is fp16, bf16 or fp32 (TF_* code).
 * Replaces exl3/linear.cpp:24-33 `rot_in`. */
int tf_exl3_rot_in(const void* x, int x_dtype, const uint16_t* suh, uint16_t* xh, int m, int k, tf_stream_t stream);
/* y[m, n] = ((xh @ W_q) @ H / sqrt(128)) * svh + bias, 1 <= m <= 128.  T: trellis words, tile (kt, nt) at
 * kt*stride_k + (nt/8)*stride_nb + (nt%8)*4*k2 words; k2 = 2*bits; cb 0 3inst, 1 mcg, 2 mul1; sk K splits (Z fp32
 * [sk, m, n] and zeroed int32 counters [8 * n/128 * TF_EXL3_COUNTER_STRIDE] needed when sk > 1 (each counter alone in
 * 64 bytes); counters are left zero); wk waves a block.
 * Replaces exl3/linear.cpp:36-58 `linear`. */
int tf_exl3_linear(const uint16_t* xh, const uint32_t* T, int64_t stride_k, int64_t stride_nb, const uint16_t* svh,
                   const uint16_t* bias, void* y, int y_dtype, float* Z, int32_t* counters, int m, int k, int n,
                   int k2, int cb, int sk, int wk, tf_stream_t stream);
/* The same two calls over a stack of 1 to 64 layers of one shape, width and codebook that read the same x (an MLP's
 * gate and up projections): one launch each instead of one a layer, every layer's bits those of its own call.
 * suh [layers, k]; xh [layers, m, k]; layer z's trellis stride_layer words past layer 0's; svh, bias [layers, n];
 * y [layers, m, n]; Z [layers, sk, m, n]; counters [layers, 8 * n/128 * TF_EXL3_COUNTER_STRIDE].  The reference's
 * linear module has no such call; its affine path groups launches the same way (kernels/qmm.cpp:51-54 `qmm_group`). */
int tf_exl3_rot_in_stacked(const void* x, int x_dtype, const uint16_t* suh, uint16_t* xh, int layers, int m, int k,
                           tf_stream_t stream);
int tf_exl3_linear_stacked(const uint16_t* xh, const uint32_t* T, int64_t stride_k, int64_t stride_nb,
                           int64_t stride_layer, const uint16_t* svh, const uint16_t* bias, void* y, int y_dtype,
                           float* Z, int32_t* counters, int layers, int m, int k, int n, int k2, int cb, int sk, int wk,
                           tf_stream_t stream);
/* An MLP's gate and up projections with the SwiGLU and the down projection's input rotation in the same launch:
 * tf_exl3_linear_stacked over two layers (gate first), in which the workgroup that completes a column block over both
 * layers' K splits also writes xh_next[m, n] = fp16(((act * suh_next) H) / sqrt(128)), act = r(r(g / (1 + exp(-g))) * u)
 * with g, u the two outputs as y_dtype holds them and r the rounding to y_dtype: the input tf_exl3_linear takes for
 * the down projection.  y [2, m, n] may be null; Z [2, sk, m, n] and counters [8 * n/128 * TF_EXL3_COUNTER_STRIDE]
 * (zero before, left zero) are needed at every sk.  tf_exl3_swiglu_rot_in is the same producer as a launch of its own
 * over a stored y [2, m, n] (same bits).  The reference's linear module has neither: its callers run the elementwise
 * steps in torch between two `linear` calls (exl3/linear.py:165-186 `__call__`); the roundings are those of its
 * other SwiGLU epilogues (kernels/qwen/flash_next/v1/base.py:35, experts.py:122). */
int tf_exl3_gate_up(const uint16_t* xh, const uint32_t* T, int64_t stride_k, int64_t stride_nb, int64_t stride_layer,
                    const uint16_t* svh, const uint16_t* bias, void* y, int y_dtype, float* Z, int32_t* counters,
                    const uint16_t* suh_next, uint16_t* xh_next, int m, int k, int n, int k2, int cb, int sk, int wk,
                    tf_stream_t stream);
int tf_exl3_swiglu_rot_in(const void* y, int y_dtype, const uint16_t* suh, uint16_t* xh, int m, int n,
                          tf_stream_t stream);
/* W[k, n] fp16 = the decoded trellis (bit-exact codebook values).  Replaces exl3/linear.cpp:61-68 `unpack`. */
int tf_exl3_unpack(const uint32_t* T, uint16_t* W, int k, int n, int64_t stride_k, int64_t stride_nb, int k2, int cb,
                   tf_stream_t stream);

/* ---- EXL3 prompt matmul (exl3/prefill.py:15-95; Triton `_gemm` in the reference) ----------------------------------- */

/* W8[k / 8][n][8] fp16 = the decoded trellis in the order an MFMA B operand is read (tf_exl3_unpack's values:
 * W8[k / 8][c][k % 8] = W[k][c]; the 8 consecutive inputs of a lane are 16 bytes, a tile's 16 columns side by side).
 * The reference decodes W_q [K, N] with `unpack` once a chunk (exl3/prefill.py:88-89). */
int tf_exl3_unpack_k8(const uint32_t* T, uint16_t* W8, int k, int n, int64_t stride_k, int64_t stride_nb, int k2,
                      int cb, tf_stream_t stream);
/* y[m, block] = ((xh[m] @ W_q[:, block]) H / sqrt(128)) * svh + bias for any m: xh fp16 [m, k] from tf_exl3_rot_in,
 * w8 from tf_exl3_unpack_k8 (k * n < 2^31), K added in order in fp32 (a row's bits do not depend on m or on the
 * rows beside it), the rotation exact in fp32.  y rows are y_stride elements apart.  Replaces exl3/prefill.py:16-44
 * `_gemm`. */
int tf_exl3_gemm(const uint16_t* xh, const uint16_t* w8, const uint16_t* svh, const uint16_t* bias, void* y, int y_dtype,
                 int64_t y_stride, int m, int k, int n, tf_stream_t stream);

/* ---- EXL3 routed experts (exl3/experts.py:173-202 `routed`; pybind `tensorfold_exl3_experts_v1`, experts.cpp:132-141) --
 * Pairs p = row * slots + slot; a pick outside [0, experts) is not a routed expert and is skipped everywhere.  The
 * pairs are grouped by tf_experts_plan (tile 16, ids up to and including `experts`): items, counts, members. */

/* out0[p] = fp16(((x[p / slots] * suh0[pick[p]]) H) / sqrt(128)), and out1 from suh1 when given: fp16 [pairs, k];
 * suh fp16 [experts, k]; x rows x_stride elements apart.  Replaces experts.cpp `rot_in` (experts.cu:96-117). */
int tf_exl3x_rot_in(const void* x, int x_dtype, int64_t x_stride, const int32_t* pick, const uint16_t* suh0,
                    const uint16_t* suh1, uint16_t* out0, uint16_t* out1, int rows, int slots, int k, int experts,
                    tf_stream_t stream);
/* z[(mat * sk + split), p, :] = the split's share of x_mat[p] @ W_q of pick[p]'s matrix `mat`, fp32 [mats * sk, pairs,
 * n]: tp int64 [experts] the address of each expert's trellis (the checkpoint's [k/16, n/16, 16 * bits] int16), k2
 * int32 [experts] its half-bits a value (2..16 even; 3, 5, 7 with codebook 2), one width per expert and matrix.
 * Replaces experts.cpp `grouped` (experts_grouped.cuh:190-284). */
int tf_exl3x_grouped(const uint16_t* x0, const uint16_t* x1, const int64_t* tp0, const int64_t* tp1, const int32_t* k2_0,
                     const int32_t* k2_1, const int32_t* items, const int32_t* counts, const int32_t* members, float* z,
                     int mats, int k, int n, int pairs, int sk, int cb, int experts, int max_items, tf_stream_t stream);
/* gate and up of a pair: splits added in order, H / sqrt(128), * svh; SwiGLU clipped at `limit` (act_mode 0 with the
 * bf16 roundings of exl3/experts.cu:141-146, 1 in fp32); xd[p] = fp16(((act * suh_d) H) / sqrt(128)), fp16 [pairs, n].
 * Replaces experts.cpp `gateup_epilogue` (experts.cu:121-157). */
int tf_exl3x_gateup_epilogue(const float* z, const int32_t* pick, const uint16_t* svh_g, const uint16_t* svh_u,
                             const uint16_t* suh_d, uint16_t* xd, int pairs, int n, int sk, int experts, float limit,
                             int act_mode, tf_stream_t stream);
/* y[p] = ((splits added in order) H / sqrt(128)) * svh_d for routed pairs, fp32 [pairs, d] (other pairs keep the
 * caller's y); with wts: out[r] = fma chain over the slots in order of wts[r, k] * y[r * slots + k], fp32 [rows, d].
 * Replaces experts.cpp `down_epilogue`, `combine` and `down_combine` (experts.cu:160-237). */
int tf_exl3x_down_combine(const float* z, const int32_t* pick, const uint16_t* svh_d, float* y, const float* wts,
                          float* out, int rows, int slots, int d, int sk, int experts, tf_stream_t stream);

/* tf_experts_plan (tile 16, at most 1,024 pairs) and tf_exl3x_rot_in in one launch: workgroup 0 groups the pairs,
 * the others rotate them (neither needs the other's result).  Replaces experts.py:173-185 (the pair sort and
 * experts.cpp `rot_in`). */
int tf_exl3x_plan_rot_in(const void* x, int x_dtype, int64_t x_stride, const int32_t* pick, const uint16_t* suh0,
                         const uint16_t* suh1, uint16_t* out0, uint16_t* out1, int rows, int slots, int k, int experts,
                         int tile, int32_t* members, int32_t* items, int32_t* counts, tf_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* TFMI_H */
