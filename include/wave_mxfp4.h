/*
 * wave_mxfp4.h - C ABI of the MI355X (gfx950) MXFP4 block-scaled GEMM library.
 *
 * The library replaces the GPU kernels the reference generates from its
 * scaled-GEMM templates together with the launch call that runs them.  Every
 * entry point takes plain device pointers, sizes and a HIP stream, validates
 * its arguments before touching HIP, never synchronises and never throws;
 * it returns 0 or a negative wave_mxfp4_status.  Work is enqueued on the given
 * stream (NULL = the default stream), like the reference's launch
 * (wave_lang/kernel/wave/runtime/runtime.cpp:123-203 called from
 * wave_lang/kernel/wave/utils/run_utils.py:62-134).
 *
 * Data formats (inputs of the drop-in API):
 *   A        [M, K/2]  uint8, two e2m1 codes per byte, low nibble first
 *   B        [N, K/2]  uint8, N-major, so C = A . B^T
 *   A_scale  [M, K/32] uint8 e8m0, one per 32 elements along K
 *   B_scale  [N, K/32] uint8 e8m0
 *   C        [M, N]    float or bf16, row-major, written in place
 * (wave_lang/kernel/wave/templates/tagged_mxfp4_gemm.py:93-122,
 *  wave_lang/kernel/wave/utils/mxfp_utils.py:20-57).
 */
#ifndef WAVE_MXFP4_H_
#define WAVE_MXFP4_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum {
  WAVE_MXFP4_OK = 0,
  WAVE_MXFP4_ERR_NULL_POINTER = -1,
  WAVE_MXFP4_ERR_BAD_SHAPE = -2,     /* negative dims, K % 32 != 0, layout divisibility */
  WAVE_MXFP4_ERR_BAD_ENUM = -3,      /* dtype / layout / variant out of range */
  WAVE_MXFP4_ERR_MISALIGNED = -4,    /* a pointer is not aligned as documented */
  WAVE_MXFP4_ERR_WORKSPACE = -5,     /* workspace missing or too small (split-K, per-row scales) */
  WAVE_MXFP4_ERR_BAD_SPLIT = -6,     /* K per split < 256 or not a multiple of 256 */
  WAVE_MXFP4_ERR_HIP = -7,           /* a HIP call failed; see wave_mxfp4_last_hip_error */
  WAVE_MXFP4_ERR_UNSUPPORTED = -8
} wave_mxfp4_status;

/* Output element type, fixed per kernel build in the reference
 * (tagged_mxfp4_gemm.py:62-65,120-122); bf16 is round-to-nearest-even of the
 * f32 accumulator. */
typedef enum { WAVE_MXFP4_OUT_F32 = 0, WAVE_MXFP4_OUT_BF16 = 1 } wave_mxfp4_out_dtype;

/* Scale storage.  ROW_MAJOR is [R, K/32].  E8M0_SHUFFLE is the tile order of
 * e8m0_shuffle (mxfp_utils.py:113-128, tagged_mxfp4_gemm.py:485-536) over a
 * buffer padded to ceil(R/32)*32 rows and ceil(K/32/8)*8 columns; the buffer
 * must hold every byte of that padded shape (the reference's final slice back
 * to [R, K/32] loses bytes unless R % 32 == 0 and K % 256 == 0). */
typedef enum {
  WAVE_MXFP4_SCALE_ROW_MAJOR = 0,
  WAVE_MXFP4_SCALE_E8M0_SHUFFLE = 1,
  /* The layout the 32x32x64 scaled MFMA kernels read with one dword per lane:
   * per 32-row tile and 256-element K tile a 256-byte block; lane
   * (g%2)*32 + r%32 holds, in byte (g%8)/2, the scale of row r, group g.  Same
   * byte count as the padded E8M0_SHUFFLE buffer.  Produced by
   * wave_mxfp4_scale_convert (no counterpart in the reference, whose
   * e8m0_shuffle is matched to the 16x16x128 instruction). */
  WAVE_MXFP4_SCALE_MFMA32 = 2,
  /* One e8m0 byte per row, [R], that holds for every 32-group of the row: the
   * broadcast-scale kernel of the reference
   * (wave_lang/kernel/wave/templates/test_kernels.py:75-135, a_scale: [M]
   * broadcast to [M, K/32]).  Accepted as a_scale_layout of wave_mxfp4_gemm
   * only; the call then needs the workspace, in which the library spreads the
   * scales out before the GEMM. */
  WAVE_MXFP4_SCALE_PER_ROW = 3
} wave_mxfp4_scale_layout;

/* B storage.  PRESHUFFLE is b_preshuffle (mxfp_utils.py:98-110,
 * tagged_mxfp4_gemm.py:465-483); needs N % 16 == 0 and K % 64 == 0. */
typedef enum { WAVE_MXFP4_B_ROW_MAJOR = 0, WAVE_MXFP4_B_PRESHUFFLE = 1 } wave_mxfp4_b_layout;

/* Element type of the quantiser's input. */
typedef enum { WAVE_MXFP4_IN_F32 = 0, WAVE_MXFP4_IN_BF16 = 1, WAVE_MXFP4_IN_F16 = 2 } wave_mxfp4_in_dtype;

/* Kernel selection.  AUTO picks by shape.  The others force one kernel and
 * mirror the reference's (block_shape, wave_shape) template arguments
 * (tagged_mxfp4_gemm.py:38-48). */
typedef enum {
  WAVE_MXFP4_VARIANT_AUTO = 0,
  WAVE_MXFP4_VARIANT_T256x256_W2x2 = 1, /* 256x256x256 tile, 4 waves */
  WAVE_MXFP4_VARIANT_T256x256_W4x2 = 2, /* 256x256x256 tile, 8 waves */
  WAVE_MXFP4_VARIANT_T128x128_W2x2 = 3, /* 128x128x256 tile, 4 waves */
  WAVE_MXFP4_VARIANT_SKINNY = 4,        /* M <= 64 streaming kernel */
  WAVE_MXFP4_VARIANT_NAIVE = 5,         /* one thread per C element, for cross-checks */
  WAVE_MXFP4_VARIANT_T128x256_W2x2 = 6, /* 128x256x256 tile, 4 waves */
  /* 256x256x256 tile, 4 waves side by side along N; A through LDS, preshuffled B
   * straight from global memory into registers: the asymmetric kernels of the
   * reference (tagged_mxfp4_gemm.py:950-991 with schedules/
   * gemm_mxfp4_double_buffer.py:1781-2222).  Needs b_layout PRESHUFFLE,
   * N % 256 == 0, K % 512 == 0, K >= 1536 and either MFMA32 scales or the
   * workspace; WAVE_MXFP4_ERR_UNSUPPORTED otherwise.  AUTO takes it where it
   * applies and the problem has more tiles than the GPU has CUs. */
  WAVE_MXFP4_VARIANT_T256x256_W1x4_BDIRECT = 7,
  /* M <= 256 against a wide B from HBM: one workgroup per strip of 64 to 128 columns, B through deep
   * wave-private LDS rings, A fed by a producer wave.  Needs K > 768, N % 4 == 0, no split, and
   * each scale tensor row-major, MFMA32 or in e8m0_shuffle order (all three read as they are, no pass per call);
   * a K that is not a multiple of 256 with both scale tensors in MFMA32 order, padding groups 0 as
   * wave_mxfp4_scale_convert and the quantiser write them (row-major ones are re-laid in the workspace first);
   * WAVE_MXFP4_ERR_UNSUPPORTED otherwise.  AUTO takes it for 16 < M <= 256 and a wide N (M <= 16 too at K <= 4096), and for a grouped problem of few rows per expert
   * (see wave_mxfp4_gemm_grouped).  The reference runs such shapes through its generic tile kernel
   * (tests/kernel/wave_gemm_mxfp_test.py:291-339). */
  WAVE_MXFP4_VARIANT_MID_M = 8,
  /* 256x192x256 tile, 8 waves, persistent kernel only: for problems whose count of 256x256 tiles leaves the last
   * round over the CUs partly empty while 256x192 tiles fill whole rounds (4093 x 6144: 384 tiles are 1.5 rounds
   * of 256 CUs, 512 tiles of 256x192 are 2 rounds of three quarters the work each).  Needs N % 192 == 0, more
   * tiles than CUs, K >= 768 and scales in MFMA32 order or the workspace; WAVE_MXFP4_ERR_UNSUPPORTED otherwise.
   * AUTO takes it when its rounds cost less.  The reference fixes one block shape per compiled kernel
   * (wave_lang/kernel/wave/templates/tagged_mxfp4_gemm.py:38-145); picking it per problem is the library's. */
  WAVE_MXFP4_VARIANT_T256x192_W4x2 = 9,
  /* M <= 256 against a wide preshuffled B from HBM: one workgroup per strip of 128 columns, 4 waves side by
   * side along N; A through an LDS ring that takes the whole LDS, B straight from global memory into registers
   * four K tiles ahead (the reference's asymmetric data flow, tagged_mxfp4_gemm.py:950-991, at a decode-sized M).
   * Needs b_layout PRESHUFFLE, M <= 256, N % 32 == 0, K % 2048 == 0 (K % 1024 == 0 from M = 129 on), no split,
   * and MFMA32 scales or the workspace; WAVE_MXFP4_ERR_UNSUPPORTED otherwise.  AUTO takes it for 128 < M <= 256
   * where it applies and N >= 12288 (below that M variant 8 is as fast on the same operands). */
  WAVE_MXFP4_VARIANT_MID_M_BDIRECT = 10,
  WAVE_MXFP4_VARIANT_COUNT_
} wave_mxfp4_variant;

/*
 * C[M,N] = dequant(A) . dequant(B)^T.
 * Replaces the compiled kernel call gemm(x, x_scales, w_t, w_scales, out)
 * (tests/kernel/wave_gemm_mxfp_test.py:194-201; kernels of
 * tagged_mxfp4_gemm.py:38-145,334-403,950-991 and the split-K family
 * :611-947) and its launch (runtime.cpp:123-203).
 *   split_k   0 = automatic, 1 = off, n > 1 = n splits along K; each split
 *             must own a multiple of 256 elements (tagged_mxfp4_gemm.py:636-645).
 *             Partial sums are kept in f32 in `workspace` and reduced in a
 *             fixed order, so C is overwritten, never accumulated into.
 *   workspace device scratch, 256-byte aligned, of wave_mxfp4_workspace_bytes(...)
 *             bytes: the split-K partial sums (required for a split) plus room
 *             to re-lay ROW_MAJOR / E8M0_SHUFFLE scales out as MFMA32 before the
 *             tile kernels run (optional: without it the kernels read the given
 *             layout directly, which costs vector-L1 time).  May be NULL.
 * A, B must be 16-byte aligned; scales 8-byte aligned; C 16-byte aligned.
 */
int wave_mxfp4_gemm(const void *a, const void *a_scale, const void *b, const void *b_scale, void *c,
                    int64_t m, int64_t n, int64_t k, int out_dtype, int a_scale_layout,
                    int b_scale_layout, int b_layout, int split_k, void *workspace,
                    size_t workspace_bytes, int variant, void *hip_stream);

/* Scratch bytes wave_mxfp4_gemm can use for (m, n, k, split_k, variant): the
 * split-K partials (for split_k == 0, of the split the library would pick by
 * itself; given less, it takes fewer parts) plus the re-laid-out scales of both
 * operands. */
size_t wave_mxfp4_workspace_bytes(int64_t m, int64_t n, int64_t k, int split_k, int variant);

/*
 * wave_mxfp4_gemm for callers that cannot allocate device memory (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc); it has
 * no counterpart in the reference.  Same arguments and results as
 * wave_mxfp4_gemm without the workspace pair: the scratch (re-laid scales,
 * split-K partial sums, the parts of a sparsely filled last round of tiles) is
 * a fixed array of wave_mxfp4_static_scratch_bytes() = 16 MiB inside the
 * library's device image, one per GPU, held until the process ends.  The call
 * allocates and frees nothing, provided wave_mxfp4_static_scratch_bytes() was
 * called once on that device beforehand (set-up: it looks the array's address
 * up, which may load the library's code object; without it the first
 * wave_mxfp4_gemm_static of a device does the lookup itself).  A problem whose
 * scratch (wave_mxfp4_workspace_bytes(m, n, k, split_k, variant), less the parts
 * this call's layouts do not use: scale tensors already in MFMA32 order are read
 * in place) exceeds that size is
 * rejected with WAVE_MXFP4_ERR_WORKSPACE (wave_mxfp4_last_hip_error() then
 * holds the two sizes); 8192^3 needs 6.3 MB.  With split_k == 0 what has to fit
 * is the call without a split: the library's own split takes as many parts as
 * the array holds beside the scales, as wave_mxfp4_gemm does with a workspace
 * of that size.  All calls on one GPU share the
 * array: calls that overlap in time on one GPU (different streams, or threads
 * without ordering) race on it; calls on one stream are ordered and safe.
 */
int wave_mxfp4_gemm_static(const void *a, const void *a_scale, const void *b, const void *b_scale, void *c,
                           int64_t m, int64_t n, int64_t k, int out_dtype, int a_scale_layout,
                           int b_scale_layout, int b_layout, int split_k, int variant, void *hip_stream);
size_t wave_mxfp4_static_scratch_bytes(void);

/*
 * Grouped (MoE) GEMM: rows offsets[e] .. offsets[e+1]-1 of A (sorted by expert)
 * are multiplied by expert e's B[e] [N, K/2] with B_scale[e]; C is
 * [total_rows, N].  `offsets` is a DEVICE array of num_groups+1 int32,
 * non-decreasing, offsets[0] = 0, offsets[num_groups] <= total_rows; empty
 * groups are allowed.  The array lives on the device, so it is clamped there,
 * not validated: each group's range is cut to [0, total_rows] with end >=
 * begin, which keeps every access inside the buffers; what a malformed array
 * computes is unspecified.  B is [E, N, K/2]; B_scale is [E, N, K/32] row-major, or
 * E shuffled buffers of ceil(N/32)*32 x ceil(K/256)*8 bytes each.
 * The reference has no grouped MXFP4 kernel: this replaces its per-expert
 * Python loop over single GEMMs (tests/kernel/moe_test.py:175-246).
 * `workspace` is optional scratch (256-byte aligned) of
 * wave_mxfp4_grouped_workspace_bytes(...) bytes: with it the scales of both
 * operands are first re-laid out for one-dword-per-lane reads, as in
 * wave_mxfp4_gemm (N % 32 == 0 and K % 256 == 0; otherwise it is not used),
 * and large problems run the persistent kernel over a table of M tiles built
 * there; a scale tensor handed over in WAVE_MXFP4_SCALE_MFMA32 order (resident
 * weights, activations from wave_mxfp4_quantize) is read where it is.  For
 * problems of at most four rounds of 256x256 tiles over the CUs the size
 * includes 256 KB per CU for the f32 parts of a sparsely filled last round,
 * whose tiles are then cut along K and summed by a second launch.
 * A small batch (AUTO: at most 160 rows per expert on average - or more where
 * the tile kernels would leave CUs idle for whole rounds, e.g. few column tiles
 * and a long K - and enough experts x 128-column strips to occupy half the CUs)
 * runs on the mid-M kernel,
 * one workgroup per (expert, strip), with no table and no scale re-layout: the
 * call is then bound by reading every expert's B once.  It needs K > 768,
 * N % 4 == 0, A's scales row-major or MFMA32 and B's in any of the three orders
 * (a K that is not a multiple of 256: both in MFMA32 order, padding groups 0);
 * WAVE_MXFP4_VARIANT_MID_M asks for it by name (WAVE_MXFP4_ERR_UNSUPPORTED
 * where it does not apply).  The other variants accepted here are AUTO, NAIVE
 * and the square tile shapes.
 */
int wave_mxfp4_gemm_grouped(const void *a, const void *a_scale, const void *b, const void *b_scale,
                            void *c, const int32_t *offsets, int num_groups, int64_t total_rows,
                            int64_t n, int64_t k, int out_dtype, int a_scale_layout,
                            int b_scale_layout, int b_layout, int variant, void *workspace,
                            size_t workspace_bytes, void *hip_stream);
size_t wave_mxfp4_grouped_workspace_bytes(int64_t total_rows, int64_t n, int64_t k, int num_groups);

/* Element format of the MXFP8 operands (OCP MX: e4m3 is the "fn" variant without
 * infinities, e5m2 is IEEE-like).  WAVE_MXFP8_E2M1 (= WAVE_MXFP8_B_E2M1, its older name) marks one operand, A or
 * B but not both, as MXFP4: [rows, K/2] packed as in wave_mxfp4_gemm, against an 8-bit other operand. */
typedef enum { WAVE_MXFP8_E4M3 = 0, WAVE_MXFP8_E5M2 = 1, WAVE_MXFP8_B_E2M1 = 2, WAVE_MXFP8_E2M1 = 2 } wave_mxfp8_format;

/* The same block-scaled GEMM on MXFP8 operands: A [M, K] of a_format and
 * B [N, K] of b_format, one byte per element (the formats may differ: cbsz /
 * blgp 0 / 1 of the instruction; WAVE_MXFP8_E2M1 for one of them: that operand [rows, K/2], two e2m1
 * per byte, cbsz / blgp 4 - the mixed operand types the reference's scaled MMA admits in either order,
 * wave_lang/kernel/wave/constraints.py:425-431; both e2m1 is wave_mxfp4_gemm's and WAVE_MXFP4_ERR_UNSUPPORTED here),
 * scales [R, K/32] e8m0 row-major,
 * C f32 or bf16.  Replaces the kernel of tests/kernel/wave_gemm_mxfp_test.py:416-501
 * (tkl.f8e5m2 operands through the same scaled MFMA).  K % 128 == 0; variant
 * AUTO, T256x256_W2x2, T256x256_W4x2 or T128x128_W2x2.  `workspace` is optional scratch of
 * wave_mxfp8_workspace_bytes(m, n, k) bytes (256-byte aligned): with it, and
 * K % 256 == 0, the scales are first re-laid out for one-dword-per-lane reads,
 * and a problem of at most 128 tiles of 128x128 with a K of 2048 or more is
 * cut along K into up to 8 parts (f32 partial tiles in the scratch, summed by
 * one more launch; C is overwritten, the sum order is fixed): 128 x 1024 x 8192
 * 65 -> 23 us.  A scratch that only holds the scales keeps K whole. */
int wave_mxfp8_gemm(const void *a, const void *a_scale, const void *b, const void *b_scale, void *c,
                    int64_t m, int64_t n, int64_t k, int a_format, int b_format, int out_dtype, void *workspace,
                    size_t workspace_bytes, int variant, void *hip_stream);
size_t wave_mxfp8_workspace_bytes(int64_t m, int64_t n, int64_t k);

/* An 8-bit B [rows, K] (one byte per element) into the order a B-direct kernel
 * reads with one coalesced 16-byte load per lane and half MFMA operand: the
 * 8-bit counterpart of b_preshuffle (mxfp_utils.py:98-110, which the
 * reference defines for packed MXFP4 rows only; this layout is this
 * library's).  Blocks of 32 rows x 128 bytes (one K tile), 4096 bytes each,
 * block (r / 32, kt) at ((r / 32) * (K / 128) + kt) * 4096; inside a block
 * the 16-byte pieces follow each other as [K step s = 0..1][half h = 0..1]
 * [lane l = 0..63], and lane l = 32 * g + r' holds row r' of the block, bytes
 * 64 * s + 32 * h + 16 * g .. + 15 of the K tile (the scaled MFMA takes a
 * lane's 32 bytes of an 8-bit operand as two halves 32 bytes apart in K).
 * rows % 32 == 0, K % 128 == 0; not in place. */
int wave_mxfp8_b_preshuffle(const void *b, void *out, int64_t rows, int64_t k, void *hip_stream);

/* wave_mxfp8_gemm with B in wave_mxfp8_b_preshuffle order: A through LDS, B
 * straight from global memory into registers (the schedule of
 * wave_lang/kernel/wave/schedules/gemm_mxfp4_double_buffer.py:1781-2222 on the
 * operands of tests/kernel/wave_gemm_mxfp_test.py:416-501).  A 8-bit (e4m3 /
 * e5m2), B 8-bit in any pairing with it, or b_format = WAVE_MXFP8_E2M1: then b
 * is packed MXFP4 [N, K/2] in wave_mxfp4_b_preshuffle order (the weights of
 * the MXFP4 B-direct kernels, here against 8-bit activations).  N % 256 == 0,
 * K % 256 == 0, K >= 768, any M; each scale tensor row-major or
 * WAVE_MXFP4_SCALE_MFMA32 (with a row-major one the workspace of
 * wave_mxfp8_workspace_bytes(m, n, k) bytes is required: it is re-laid out
 * there first).  WAVE_MXFP4_ERR_UNSUPPORTED otherwise. */
int wave_mxfp8_gemm_b_preshuffled(const void *a, const void *a_scale, const void *b, const void *b_scale, void *c,
                                  int64_t m, int64_t n, int64_t k, int a_format, int b_format, int out_dtype,
                                  int a_scale_layout, int b_scale_layout, void *workspace, size_t workspace_bytes,
                                  void *hip_stream);

/* Packed e2m1 [rows, kp] -> f32 [rows, 2*kp] through the 16-entry table, code 8
 * gives -0.0 (mxfp_utils.py:60-83).  Bit-exact. */
int wave_mxfp4_to_f32(const void *q, float *out, int64_t rows, int64_t kp, void *hip_stream);

/* e8m0 bytes -> f32 2^(s-127), 255 -> NaN, 0 -> 2^-127 (mxfp_utils.py:86-95).
 * Bit-exact. */
int wave_mxfp4_e8m0_to_f32(const void *s, float *out, int64_t count, void *hip_stream);

/* out[r, e] = value(q[r, e]) * scale(r, e / 32), f32, the operand the reference
 * feeds to its matmul (mxfp_utils.py:135-143).  Bit-exact. */
int wave_mxfp4_dequant(const void *q, const void *scale, float *out, int64_t rows, int64_t k,
                       int scale_layout, void *hip_stream);

/* Device-side e8m0_shuffle (mxfp_utils.py:113-128) into the padded buffer of
 * ceil(rows/32)*32 x ceil(ks/8)*8 bytes (padding bytes written as 0). */
int wave_mxfp4_e8m0_shuffle(const void *scale, void *out, int64_t rows, int64_t ks, void *hip_stream);
size_t wave_mxfp4_e8m0_shuffle_bytes(int64_t rows, int64_t ks);

/* Re-lays a scale tensor out from one wave_mxfp4_scale_layout to another
 * (device side; generalises e8m0_shuffle, mxfp_utils.py:113-128).  Non row-major
 * buffers hold wave_mxfp4_e8m0_shuffle_bytes(rows, ks) bytes; padding is
 * written as 0. */
int wave_mxfp4_scale_convert(const void *src, int src_layout, void *dst, int dst_layout, int64_t rows,
                             int64_t ks, void *hip_stream);

/* Device-side b_preshuffle (mxfp_utils.py:98-110); rows % 16 == 0, kp % 32 == 0. */
int wave_mxfp4_b_preshuffle(const void *b, void *out, int64_t rows, int64_t kp, void *hip_stream);

/* Activation / weight quantiser, the step in front of the GEMM:
 * x [rows, k] (f32, bf16 or f16, row-major, 16-byte aligned) -> q [rows, k/2]
 * packed e2m1 + one e8m0 scale per 32 elements of a row, written in
 * `scale_layout` (row-major [rows, k/32], or a tiled layout over the padded
 * buffer of wave_mxfp4_e8m0_shuffle_bytes(rows, k/32) bytes, padding written
 * as 0), so that its outputs are the GEMM's A and A_scale (or B and B_scale)
 * without a pass in between.  k % 32 == 0.
 * Replaces aiter.get_triton_quant(QuantType.per_1x32)(x, shuffle=...) at the
 * reference's call sites (wave_lang/kernel/wave/perf/bench_mxfp4_comparison.py:
 * 1484-1486,1897-1899; shuffle=True is WAVE_MXFP4_SCALE_E8M0_SHUFFLE): scale
 * 2^(floor(log2(amax rounded up at 1.75 of a binade)) - 2) clamped to
 * 2^-127..2^127, elements rounded to nearest even, saturating at 6; NaN
 * elements become +-6 under scale byte 254. */
int wave_mxfp4_quantize(const void *x, int in_dtype, void *q, void *scale, int64_t rows, int64_t k,
                        int scale_layout, void *hip_stream);

/* The quantiser over gathered rows: output row r is the quantised row
 * row_ids[r] / row_div of x [src_rows, k]; an id at or beyond src_rows * row_div
 * (the padding value of wave_mxfp4_moe_align_block_size) gives a row of zeros
 * with scale bytes 0.  With row_ids = sorted_ids and row_div = top_k this is the
 * reference's per-expert gather of the repeated activations,
 * a.view(m, -1, k).repeat(1, topk, 1)[mask] (tests/kernel/moe_test.py:113-127),
 * fused into the quantiser: its outputs are the grouped GEMM's A and A_scale. */
int wave_mxfp4_quantize_rows(const void *x, int in_dtype, int64_t src_rows, const int32_t *row_ids, int row_div,
                             void *q, void *scale, int64_t rows, int64_t k, int scale_layout, void *hip_stream);

/* Token alignment by expert, moe_align_block_size of the reference
 * (tests/kernel/moe/torch_kernels.py:10-92): topk_ids holds num_entries =
 * num_tokens * top_k expert ids (int32, or int64 as torch.topk returns them:
 * ids_int64 = 1).  sorted_ids[sorted_len] receives, expert by expert, the flat
 * indices of the entries routed to that expert in increasing order, each
 * expert's run padded to a multiple of block_size with the value num_entries,
 * which also fills the buffer past the padded total; expert_ids[b] the expert
 * of block b below the padded total / block_size; num_tokens_post_pad[0] the
 * padded total.  expert_offsets (may be NULL) receives the num_experts + 1
 * running sums of the padded counts: with block_size = 1 they are the `offsets`
 * argument of wave_mxfp4_gemm_grouped over the sorted rows (not an output of
 * the reference function).  Ids outside [0, num_experts) are skipped.
 * num_experts <= 1024; sorted_len >= num_entries. */
int wave_mxfp4_moe_align_block_size(const void *topk_ids, int ids_int64, int64_t num_entries, int num_experts,
                                    int block_size, int32_t *sorted_ids, int64_t sorted_len, int32_t *expert_ids,
                                    int64_t expert_ids_len, int32_t *num_tokens_post_pad, int32_t *expert_offsets,
                                    void *hip_stream);

/* out = gate * up / (1 + exp(-gate)), the gated activation between the two
 * expert GEMMs (silu_and_mul_ref, tests/kernel/moe_test.py:39-40; kernel
 * wave_lang/kernel/wave/templates/moe.py:89-145).  gate, up, out are
 * [rows, n] of dtype WAVE_MXFP4_IN_BF16 or WAVE_MXFP4_IN_F16 with row strides
 * ld_* in elements (so the two halves of a [rows, 2n] GEMM output can be
 * passed as gate = x, up = x + n, ld = 2n); computed in f32, rounded once.
 * n and the strides are multiples of 8, pointers 16-byte aligned. */
int wave_mxfp4_silu_and_mul(const void *gate, const void *up, void *out, int64_t ld_gate, int64_t ld_up,
                            int64_t ld_out, int dtype, int64_t rows, int64_t n, void *hip_stream);

/* The same activation fused into the quantiser: q, scale = quantise(round to
 * dtype(silu(gate) * up)), bit-identical to wave_mxfp4_silu_and_mul followed
 * by wave_mxfp4_quantize without the [rows, n] round trip through memory.
 * n % 32 == 0. */
int wave_mxfp4_silu_and_mul_quantize(const void *gate, const void *up, int64_t ld_gate, int64_t ld_up, int dtype,
                                     void *q, void *scale, int64_t rows, int64_t n, int scale_layout,
                                     void *hip_stream);

/* The first GEMM of a gated expert MLP with the activation and the quantiser of
 * the second GEMM's operand fused into its C write: the reference's chain
 * "gate/up GEMM -> silu_and_mul -> (quantise) -> down GEMM"
 * (tests/kernel/moe_test.py:113-129; templates/test_kernels.py:74 notes the fused
 * dynamic quantisation as not done there).  b [num_groups, 2 I, K/2] and its
 * scales hold each expert's gate projection [I, K] and up projection [I, K]
 * INTERLEAVED in blocks of 32 rows (wave_mxfp4_interleave_gate_up, once per
 * weight); n = 2 I.  Instead of C [total_rows, n] the call writes
 * q [total_rows, I / 2] packed e2m1 and scale (e8m0 per row and 32 columns,
 * act_scale_layout = WAVE_MXFP4_SCALE_MFMA32, the order the second GEMM reads) of
 * silu(gate) * up, bit-identical to wave_mxfp4_gemm_grouped (bf16 out) followed
 * by wave_mxfp4_silu_and_mul_quantize on its two halves.  num_groups = 0 with
 * offsets = NULL is the dense problem.  Served by two kernels: the persistent
 * 256x256 kernel (more 256x256 tiles than CUs), and, for a small batch routed
 * over the experts (grouped, the batches wave_mxfp4_gemm_grouped gives to the
 * mid-M kernel: at most 160 rows per expert on average and some beyond, the
 * experts' B scales resident in MFMA32 order, at least half as many
 * 128-column strips over all experts as CUs), the mid-M kernel that
 * wave_mxfp4_gemm_grouped gives such a batch to, on the same block height.  Either way I % 128 == 0,
 * K % 256 == 0, K >= 1024 (768 on the persistent kernel), a workspace of
 * wave_mxfp4_grouped_workspace_bytes(total_rows, n, k, max(num_groups, 1)) bytes,
 * scales row-major or MFMA32, B row-major; WAVE_MXFP4_ERR_UNSUPPORTED
 * otherwise (the caller then runs the two calls).  Rows past the last offset
 * are left untouched, as are the padding rows of an MFMA32 scale tensor. */
int wave_mxfp4_gemm_gated_quantize(const void *a, const void *a_scale, const void *b, const void *b_scale, void *q,
                                   void *scale, const int32_t *offsets, int num_groups, int64_t total_rows, int64_t n,
                                   int64_t k, int a_scale_layout, int b_scale_layout, int act_scale_layout,
                                   void *workspace, size_t workspace_bytes, void *hip_stream);

/* Row interleave for wave_mxfp4_gemm_gated_quantize: src is [2 * half_rows,
 * row_bytes] bytes, gate rows first, up rows behind them (packed weights
 * [2 I, K/2] or their row-major scales [2 I, K/32]); dst receives blocks of 32
 * rows alternating gate, up, gate, ...  half_rows % 32 == 0.  (No counterpart
 * in the reference, which keeps the two projections apart.) */
int wave_mxfp4_interleave_gate_up(const void *src, void *dst, int64_t half_rows, int64_t row_bytes, void *hip_stream);

/* Text for a status code; never NULL (the reference reports errors as
 * exceptions carrying hipGetErrorName/String, runtime.cpp:96-109). */
const char *wave_mxfp4_status_string(int status);

/* Name and text of the last HIP error this thread hit inside the library. */
const char *wave_mxfp4_last_hip_error(void);

/* Library ABI version (bumped on any signature change). */
int wave_mxfp4_abi_version(void);

#ifdef __cplusplus
}
#endif
#endif /* WAVE_MXFP4_H_ */
