// Shared declarations of the gfx950 MXFP4 GEMM library (device helpers, the
// kernel parameter block, launcher prototypes).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/wave_mxfp4.h"

namespace wave_mxfp4 {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v2f __attribute__((ext_vector_type(2)));
typedef unsigned short v4us __attribute__((ext_vector_type(4)));

#define WAVE_LDS_PTR(p) ((__attribute__((address_space(3))) void *)(p))
#define WAVE_GLOBAL_PTR(p) ((const __attribute__((address_space(1))) void *)(p))

// One K tile is 256 elements = 128 packed bytes = 8 chunks of 16 bytes (one
// chunk is the 32 elements a lane feeds to one scaled MFMA) = 8 scale groups.
constexpr int kTileK = 256;
constexpr int kTileKBytes = 128;

// Parameter block of the tile, skinny and naive GEMM kernels.
struct GemmParams {
  const uint8_t *a;        // [M, kp]
  const uint8_t *a_scale;  // row-major [M, ks] or shuffled
  const uint8_t *b;        // [E, N, kp] (E = 1 unless grouped)
  const uint8_t *b_scale;  // [E, N, ks] or E shuffled buffers
  void *c;                 // [M, N] f32 / bf16
  float *partial;          // split-K slices [splits, M, N] f32, or null
  const int32_t *offsets;  // grouped: device [E+1]; else null
  const int32_t *tile_table;  // grouped, persistent kernel: device table of M tiles (int32 x 4 each: entry 0 =
                              // {tiles, full tiles}, entry 1 + t = {first row, rows, expert, band}: mxfp4_group_table.h)
  int m, n, k;
  int kp;              // K / 2
  int ks;              // K / 32
  int ksp;             // padded scale row length of the shuffled layout: ceil(ks/8)*8
  int k_tiles;         // ceil(K / 256)
  int tiles_per_split; // K tiles owned by one split
  int splits;
  int out_bf16;
  int a_scale_layout, b_scale_layout;  // wave_mxfp4_scale_layout
  int b_preshuffled;
  int tail_parts;      // persistent kernel: the tiles of the last, partly filled round are cut along K into this
                       // many parts (1 = not), one part per workgroup, summed afterwards from tail_partial
  float *tail_partial; // [tiles of the last round][tail_parts][256][256] f32
  int num_groups;      // 0 = dense
  int tiles_m, tiles_n;
  int64_t b_group_stride;        // bytes between experts in b
  int64_t b_scale_group_stride;  // bytes between experts in b_scale
  uint8_t *epi_scale;            // gated epilogue: the activation's e8m0 scales (c then holds its packed codes)
  int epi_scale_layout;          // ... their layout (MFMA32)
};

// e2m1 code -> f32.  Bit 3 is the sign; codes 0..7 are 0, .5, 1, 1.5, 2, 3, 4, 6.
__device__ __forceinline__ float e2m1_to_f32(uint32_t code) {
  const uint32_t mag = code & 7u;
  // magnitudes as f32 bit patterns: exponent/mantissa follow the e2m1 fields
  // (e = mag >> 1, m = mag & 1): e == 0 -> m * 0.5, else 2^(e-1) * (1 + m/2)
  const uint32_t e = mag >> 1, mnt = mag & 1u;
  uint32_t bits = e == 0 ? (mnt ? 0x3F000000u : 0u) : (((126u + e) << 23) | (mnt << 22));
  bits |= (code & 8u) << 28;
  return __uint_as_float(bits);
}

// e8m0 byte -> f32: 2^(s-127); 0 -> 2^-127 (subnormal); 255 -> NaN.
__device__ __forceinline__ float e8m0_to_f32(uint32_t s) {
  const uint32_t bits = s == 255u ? 0x7FC00000u : (s == 0u ? 0x00400000u : (s << 23));
  return __uint_as_float(bits);
}

// f32 -> bf16 bits, round to nearest even, NaN kept quiet.
__device__ __forceinline__ uint16_t f32_to_bf16_rne(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x40u);
  u += 0x7FFFu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

// Byte offset of scale (row r, group g) in the e8m0_shuffle tile order with
// padded row length ksp.
__device__ __host__ __forceinline__ int64_t e8m0_shuffle_offset(int64_t r, int64_t g, int64_t ksp) {
  return (r >> 5) * ((ksp >> 3) * 256) + (g >> 3) * 256 + (g & 3) * 64 + (r & 15) * 4 +
         ((g & 7) >> 2) * 2 + ((r & 31) >> 4);
}

// Byte offset of scale (row r, group g) in the library's MFMA32 order: per 32-row
// tile and K tile (8 groups) one 256-byte block holding, for the lane
// (g%2)*32 + r%32 of the 32x32x64 scaled MFMA, the four bytes of its K steps
// t = (g%8)/2 = 0..3.
__device__ __host__ __forceinline__ int64_t mfma32_scale_offset(int64_t r, int64_t g, int64_t k_tiles) {
  return ((r >> 5) * k_tiles + (g >> 3)) * 256 + (((g & 1) << 5) | (r & 31)) * 4 + ((g & 7) >> 1);
}

// Byte offset of scale (r, g) for any wave_mxfp4_scale_layout.
__device__ __host__ __forceinline__ int64_t scale_offset(int layout, int64_t r, int64_t g, int64_t ks,
                                                         int64_t ksp) {
  if (layout == WAVE_MXFP4_SCALE_E8M0_SHUFFLE) return e8m0_shuffle_offset(r, g, ksp);
  if (layout == WAVE_MXFP4_SCALE_MFMA32) return mfma32_scale_offset(r, g, ksp >> 3);
  return r * ks + g;
}

// Byte offset of packed byte (row n, byte kb) in the b_preshuffle order.
__device__ __host__ __forceinline__ int64_t b_preshuffle_offset(int64_t n, int64_t kb, int64_t kp) {
  return (n >> 4) * 16 * kp + (kb >> 5) * 512 + ((kb >> 4) & 1) * 256 + (n & 15) * 16 + (kb & 15);
}

// ---- launchers (defined in the .hip files, called from the C ABI) ----
hipError_t launch_tile_gemm(const GemmParams &p, int variant, hipStream_t stream);
// hipFuncSetAttribute(MaxDynamicSharedMemorySize) once per kernel and device: the attribute belongs to the
// device's copy of the kernel.  `once` is a static of the calling launcher (one per kernel instantiation); two
// threads that both find it unset both set the attribute, which is idempotent.
constexpr int kMaxDevices = 64;
struct LdsAttrOnce {
  bool done[kMaxDevices] = {};
};
inline hipError_t allow_dynamic_lds(LdsAttrOnce &once, const void *kernel, int bytes) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  const bool tracked = dev >= 0 && dev < kMaxDevices;
  if (tracked && once.done[dev]) return hipSuccess;
  e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
  if (e == hipSuccess && tracked) once.done[dev] = true;
  return e;
}

hipError_t launch_tile_gemm_fp8(const GemmParams &p, int variant, int a_fmt, int b_fmt, hipStream_t stream);
bool persist_gemm_applies(const GemmParams &p, int variant, int num_cus);
hipError_t launch_persist_gemm(const GemmParams &p, int variant, int num_cus, hipStream_t stream);
bool persist_gemm_fp8_applies(const GemmParams &p, int num_cus);
hipError_t launch_persist_gemm_fp8(const GemmParams &p, int num_cus, int a_fmt, int b_fmt, hipStream_t stream);
bool persist_prefers_192(const GemmParams &p, int num_cus, int parts256);
bool persist_192_over_tile_kernel(const GemmParams &p, int num_cus);
bool persist_gated_applies(const GemmParams &p, int num_cus);
hipError_t launch_persist_gated(const GemmParams &p, int num_cus, hipStream_t stream);
hipError_t launch_interleave_rows(const uint8_t *src, uint8_t *dst, int64_t half_rows, int64_t row_bytes, int block,
                                  hipStream_t stream);
bool asym8_gemm_applies(const GemmParams &p, int num_cus);
hipError_t launch_asym8_gemm(const GemmParams &p, int num_cus, int a_fmt, int b_fmt, hipStream_t stream);
hipError_t launch_b8_preshuffle(const uint8_t *b, uint8_t *out, int64_t rows, int64_t k, hipStream_t stream);
bool asym_gemm_applies(const GemmParams &p, int num_cus, bool forced);
hipError_t launch_asym_gemm(const GemmParams &p, int num_cus, hipStream_t stream);
bool midb_gemm_applies(const GemmParams &p);
hipError_t launch_midb_gemm(const GemmParams &p, hipStream_t stream);
bool mid_gemm_applies(const GemmParams &p);
hipError_t launch_mid_gemm(const GemmParams &p, int num_cus, hipStream_t stream, int bm = 0);
bool mid_grouped_applies(const GemmParams &p);
bool mid_gated_applies(const GemmParams &p);
hipError_t launch_mid_gated(const GemmParams &p, int num_cus, hipStream_t stream, int bm);
int mid_max_m();
int persist_tail_parts(const GemmParams &p, int variant, int num_cus, size_t *partial_bytes);
hipError_t launch_skinny_gemm(const GemmParams &p, hipStream_t stream);
hipError_t launch_scale_spread_rows(const uint8_t *src, uint8_t *dst, int64_t rows, int64_t ks, hipStream_t stream);
hipError_t launch_quantize(const void *x, int in_dtype, const int32_t *row_ids, int row_div, int64_t src_rows,
                           uint8_t *q, uint8_t *scale, int64_t rows, int64_t k, int scale_layout, int num_cus,
                           hipStream_t stream);
hipError_t launch_silu_and_mul_quantize(const void *gate, const void *up, int64_t ld_gate, int64_t ld_up, int in_dtype,
                                        uint8_t *q, uint8_t *scale, int64_t rows, int64_t n, int scale_layout,
                                        int num_cus, hipStream_t stream);
hipError_t launch_silu_and_mul(const void *gate, const void *up, void *out, int64_t ld_gate, int64_t ld_up,
                               int64_t ld_out, int in_dtype, int64_t rows, int64_t n, hipStream_t stream);
constexpr int kMoeMaxExperts = 1024;  // experts the alignment kernel keeps counters for in LDS
hipError_t launch_moe_align(const void *topk_ids, int ids_int64, int64_t n, int num_experts, int block_size,
                            int32_t *sorted_ids, int64_t sorted_len, int32_t *expert_ids, int64_t expert_ids_len,
                            int32_t *total, int32_t *offsets, hipStream_t stream);
hipError_t launch_stream_gemm(const GemmParams &p, int num_cus, hipStream_t stream);
int stream_max_k_tiles();
hipError_t launch_naive_gemm(const GemmParams &p, hipStream_t stream);
hipError_t launch_splitk_reduce(const float *partial, void *c, int64_t mn, int splits, int out_bf16,
                                hipStream_t stream);
hipError_t launch_to_f32(const uint8_t *q, float *out, int64_t rows, int64_t kp, hipStream_t stream);
hipError_t launch_e8m0_to_f32(const uint8_t *s, float *out, int64_t count, hipStream_t stream);
hipError_t launch_dequant(const uint8_t *q, const uint8_t *scale, float *out, int64_t rows, int64_t k,
                          int scale_layout, hipStream_t stream);
hipError_t launch_scale_convert(const uint8_t *src, int src_layout, uint8_t *dst, int dst_layout, int64_t rows,
                                int64_t ks, hipStream_t stream);
hipError_t launch_e8m0_shuffle(const uint8_t *scale, uint8_t *out, int64_t rows, int64_t ks,
                               hipStream_t stream);
// What the builder of a grouped GEMM's M tile table takes (mxfp4_group_table.h); table == nullptr: none to build.
struct GroupTableArgs {
  const int32_t *offsets;
  int num_groups, bm;
  int short_rows;  // a group's last tile of at most this many rows goes to the table's short tiles (0: none do)
  int total_rows;
  int32_t *table;
};
// (with `table`, the launch's first workgroup also builds the M tile table of a grouped GEMM; a_rows == 0: B alone)
hipError_t launch_scale_pair_to_mfma32(const uint8_t *a_src, uint8_t *a_dst, int64_t a_rows, const uint8_t *b_src,
                                       uint8_t *b_dst, int64_t b_rows, int64_t ks, hipStream_t stream,
                                       const GroupTableArgs *table = nullptr);
hipError_t launch_scale_pair_shuffle_to_mfma32(const uint8_t *a_src, uint8_t *a_dst, int64_t a_rows, const uint8_t *b_src,
                                               uint8_t *b_dst, int64_t b_rows, int64_t ks, hipStream_t stream);
hipError_t launch_grouped_tile_table(const int32_t *offsets, int num_groups, int bm, int short_rows, int64_t total_rows,
                                     int32_t *table, hipStream_t stream);
hipError_t launch_b_preshuffle(const uint8_t *b, uint8_t *out, int64_t rows, int64_t kp,
                               hipStream_t stream);

// Tile geometry of a variant (0 if the variant is not a tile kernel).
void tile_variant_shape(int variant, int *bm, int *bn);
int skinny_max_m();

}  // namespace wave_mxfp4
