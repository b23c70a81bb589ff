// Activation quantiser in front of the MXFP4 GEMM (gfx950): f32 / bf16 / f16
// [rows, k] -> packed e2m1 [rows, k/2] + one e8m0 scale per 32 elements, written
// in any of the GEMM's scale layouts.  HBM bound: the input is read once with
// 16-byte loads that walk rows contiguously, the packed output is written once
// with dword stores that do the same, and the scale bytes of a workgroup's tile
// are gathered in LDS and written as whole dwords in the order of the layout.
//
// Arithmetic: the scale is taken from the group's largest magnitude, rounded up
// to the next binade when its mantissa is at least 1.75, minus two binades; the
// elements are divided by it and rounded to e2m1 (nearest, ties to even,
// saturating at 6) by v_cvt_scalef32_pk_fp4_*, two elements per instruction.
#include "mxfp4_common.h"

namespace wave_mxfp4 {

namespace {

typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

constexpr int kQuantRows = 32;  // rows of a workgroup's tile (one block of the tiled scale layouts)

// Largest of the four lanes of a quad.
__device__ __forceinline__ uint32_t quad_max(uint32_t v) {
  v = max(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0xB1, 0xF, 0xF, true));  // quad_perm [1,0,3,2]
  v = max(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x4E, 0xF, 0xF, true));  // quad_perm [2,3,0,1]
  return v;
}

// f32 bit pattern of a group's largest magnitude -> e8m0 byte.
__device__ __forceinline__ uint32_t scale_byte_of(uint32_t amax_bits) {
  const uint32_t e = (amax_bits + 0x200000u) >> 23;  // up to 256: a NaN with a large mantissa carries out of the field
  return e >= 255u ? 254u : (e > 2u ? e - 2u : 0u);
}

// The lane's 8 consecutive elements: DW dwords.
template <int DT>
struct Elems {
  static constexpr int kBytes = DT == WAVE_MXFP4_IN_F32 ? 4 : 2;
  static constexpr int kDwords = 2 * kBytes;
  uint32_t d[kDwords];

  __device__ __forceinline__ void load(const uint8_t *p, bool ok) {
#pragma unroll
    for (int i = 0; i < kDwords / 4; ++i) {
      v4i v = {0, 0, 0, 0};
      // read once: 16-bit inputs bypass the caches; an f32 lane's two loads share lines and are faster through them
      if (ok) v = kBytes == 2 ? __builtin_nontemporal_load((const v4i *)(p + 16 * i)) : *(const v4i *)(p + 16 * i);
      d[4 * i + 0] = v.x, d[4 * i + 1] = v.y, d[4 * i + 2] = v.z, d[4 * i + 3] = v.w;
    }
  }

  // f32 bit pattern of the largest magnitude (NaN patterns compare above infinity)
  __device__ __forceinline__ uint32_t amax_bits() const {
    if constexpr (DT == WAVE_MXFP4_IN_F32) {
      uint32_t m = 0;
#pragma unroll
      for (int i = 0; i < kDwords; ++i) m = max(m, d[i] & 0x7FFFFFFFu);
      return m;
    }
    uint32_t lo = 0, hi = 0;
#pragma unroll
    for (int i = 0; i < kDwords; ++i) {
      lo = max(lo, d[i] & 0x7FFFu);
      hi = max(hi, (d[i] >> 16) & 0x7FFFu);
    }
    const uint32_t h = max(lo, hi);
    if constexpr (DT == WAVE_MXFP4_IN_BF16) return h << 16;
    return __builtin_bit_cast(uint32_t, (float)__builtin_bit_cast(_Float16, (uint16_t)h));
  }

  // 8 e2m1 codes, element j in nibble j
  __device__ __forceinline__ uint32_t convert(float scale) const {
    uint32_t r = 0;
    if constexpr (DT == WAVE_MXFP4_IN_F32) {
      r = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(r, __builtin_bit_cast(float, d[0]), __builtin_bit_cast(float, d[1]), scale, 0);
      r = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(r, __builtin_bit_cast(float, d[2]), __builtin_bit_cast(float, d[3]), scale, 1);
      r = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(r, __builtin_bit_cast(float, d[4]), __builtin_bit_cast(float, d[5]), scale, 2);
      r = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(r, __builtin_bit_cast(float, d[6]), __builtin_bit_cast(float, d[7]), scale, 3);
    } else if constexpr (DT == WAVE_MXFP4_IN_BF16) {
      r = __builtin_amdgcn_cvt_scalef32_pk_fp4_bf16(r, __builtin_bit_cast(bf16x2, d[0]), scale, 0);
      r = __builtin_amdgcn_cvt_scalef32_pk_fp4_bf16(r, __builtin_bit_cast(bf16x2, d[1]), scale, 1);
      r = __builtin_amdgcn_cvt_scalef32_pk_fp4_bf16(r, __builtin_bit_cast(bf16x2, d[2]), scale, 2);
      r = __builtin_amdgcn_cvt_scalef32_pk_fp4_bf16(r, __builtin_bit_cast(bf16x2, d[3]), scale, 3);
    } else {
      r = __builtin_amdgcn_cvt_scalef32_pk_fp4_f16(r, __builtin_bit_cast(f16x2, d[0]), scale, 0);
      r = __builtin_amdgcn_cvt_scalef32_pk_fp4_f16(r, __builtin_bit_cast(f16x2, d[1]), scale, 1);
      r = __builtin_amdgcn_cvt_scalef32_pk_fp4_f16(r, __builtin_bit_cast(f16x2, d[2]), scale, 2);
      r = __builtin_amdgcn_cvt_scalef32_pk_fp4_f16(r, __builtin_bit_cast(f16x2, d[3]), scale, 3);
    }
    return r;
  }
};

// What one quantiser launch reads and writes.
struct QuantParams {
  const uint8_t *x;        // [src_rows, ld_x] elements; with `up`, the gate operand
  const uint8_t *up;       // null, or the second operand of the gated activation silu(x) * up
  const int32_t *row_ids;  // null, or for each output row the id of its source: row_ids[r] / row_div
  uint8_t *q;              // [rows, k/2]
  uint8_t *scale;
  int64_t ld_x, ld_up;     // row strides of x and up in elements
  int rows, k;
  int src_rows;            // rows of x (a row id at or beyond src_rows * row_div yields a zero row)
  int row_div;
  int scale_layout;
};

// silu(g) * u in f32, rounded to the 16-bit storage type (the value the unfused
// pipeline would have stored between its two kernels).  Hardware exp2 and
// reciprocal (about 1 ulp of f32 each, far below the 8 or 11 bits that are kept):
// the accurate expf and IEEE division cost more than the memory time of the
// kernel.
template <int DT>
__device__ __forceinline__ uint32_t gated_pair(uint32_t g2, uint32_t u2) {
  float g[2], u[2], r[2];
  if constexpr (DT == WAVE_MXFP4_IN_BF16) {
    g[0] = __builtin_bit_cast(float, g2 << 16), g[1] = __builtin_bit_cast(float, g2 & 0xFFFF0000u);
    u[0] = __builtin_bit_cast(float, u2 << 16), u[1] = __builtin_bit_cast(float, u2 & 0xFFFF0000u);
  } else {
    const f16x2 gh = __builtin_bit_cast(f16x2, g2), uh = __builtin_bit_cast(f16x2, u2);
    g[0] = (float)gh.x, g[1] = (float)gh.y, u[0] = (float)uh.x, u[1] = (float)uh.y;
  }
#pragma unroll
  for (int i = 0; i < 2; ++i)
    r[i] = g[i] * u[i] * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(g[i] * -1.44269504088896340736f));
  if constexpr (DT == WAVE_MXFP4_IN_BF16) {
    const bf16x2 o = {(__bf16)r[0], (__bf16)r[1]};
    return __builtin_bit_cast(uint32_t, o);
  } else {
    const f16x2 o = {(_Float16)r[0], (_Float16)r[1]};
    return __builtin_bit_cast(uint32_t, o);
  }
}

// A workgroup of four waves takes 32 rows x TC K tiles (TC*256 columns); a wave
// takes 8 of the rows.  Four lanes share a scale group (8 elements each); the 16
// quads of a wave take 16 consecutive groups of a row per pass, so that one load
// instruction covers up to 1 KB (bf16) and one store 256 B of a row.
// GATED: the elements are silu(x) * up of two 16-bit operands.
template <int DT, int TC, bool GATED>
__global__ void __launch_bounds__(256) quantize_kernel(const QuantParams p) {
  constexpr int kEb = Elems<DT>::kBytes;
  constexpr int kGroups = 8 * TC;              // scale groups of a tile row
  constexpr int kPasses = 8 * kGroups / 16;    // per wave: 8 rows x kGroups groups, 16 per pass
  constexpr int kBatch = DT == WAVE_MXFP4_IN_F32 || GATED ? 4 : 8;  // passes whose loads are in flight together
  static_assert(kPasses % kBatch == 0 || kPasses < kBatch, "passes come in whole batches");
  static_assert(!GATED || DT != WAVE_MXFP4_IN_F32, "the gated activation takes 16-bit operands");
  constexpr int kB = kPasses < kBatch ? kPasses : kBatch;
  __shared__ uint32_t tile_scales[kQuantRows * kGroups / 4];
  uint8_t *tile_bytes = (uint8_t *)tile_scales;

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int quad = lane >> 2, sub = lane & 3;
  const int rows = p.rows, k = p.k, scale_layout = p.scale_layout;
  const int ks = k >> 5, ksp = (ks + 7) & ~7;
  const int col_tiles = (ks + kGroups - 1) / kGroups;
  const int row_tile = blockIdx.x / col_tiles, col_tile = blockIdx.x - row_tile * col_tiles;
  const int row0 = row_tile * kQuantRows, g0 = col_tile * kGroups;

  // gathered rows: the ids of the wave's 8 rows, one per lane, fetched once (a load per unit would put two
  // dependent memory round trips in front of every batch)
  // ... and divided once: wave_src is the source row, or one past the last for "no such row"
  uint32_t wave_src = (uint32_t)p.src_rows;
  if (p.row_ids != nullptr && lane < 8 && row0 + wave * 8 + lane < rows)
    wave_src = min((uint32_t)p.row_ids[row0 + wave * 8 + lane] / (uint32_t)p.row_div, (uint32_t)p.src_rows);

  for (int pb = 0; pb < kPasses; pb += kB) {
    Elems<DT> e[kB], eu[GATED ? kB : 1];
    int lrow[kB], lgrp[kB];
#pragma unroll
    for (int i = 0; i < kB; ++i) {
      const int u = (pb + i) * 16 + quad;  // unit of the wave: (row, group)
      lrow[i] = wave * 8 + u / kGroups;
      lgrp[i] = u % kGroups;
      const int row = row0 + lrow[i], g = g0 + lgrp[i];
      bool ok = row < rows && g < ks;
      int64_t src = row;
      if (p.row_ids) {  // gathered rows
        src = (uint32_t)__shfl((int)wave_src, u / kGroups, 64);
        ok = ok && src < p.src_rows;
      }
      const int64_t col = (int64_t)g * 32 + sub * 8;
      e[i].load(p.x + (src * p.ld_x + col) * kEb, ok);
      if constexpr (GATED) eu[i].load(p.up + (src * p.ld_up + col) * kEb, ok);
    }
#pragma unroll
    for (int i = 0; i < kB; ++i) {
      const int row = row0 + lrow[i], g = g0 + lgrp[i];
      if constexpr (GATED) {
#pragma unroll
        for (int w = 0; w < Elems<DT>::kDwords; ++w) e[i].d[w] = gated_pair<DT>(e[i].d[w], eu[i].d[w]);
      }
      const uint32_t sb = scale_byte_of(quad_max(e[i].amax_bits()));
      const float sf = __builtin_bit_cast(float, sb ? sb << 23 : 0x00400000u);  // 2^(sb-127)
      const uint32_t codes = e[i].convert(sf);
      if (row < rows && g < ks) __builtin_nontemporal_store(codes, (uint32_t *)(p.q + (int64_t)row * (k >> 1) + g * 16 + sub * 4));
      if (sub == 0) {
        const int at = scale_layout == WAVE_MXFP4_SCALE_ROW_MAJOR
                           ? lrow[i] * kGroups + lgrp[i]
                           : (lgrp[i] >> 3) * 256 + (int)scale_offset(scale_layout, lrow[i], lgrp[i] & 7, 8, 8);
        tile_bytes[at] = (uint8_t)sb;
      }
    }
  }
  __syncthreads();

  uint8_t *scale = p.scale;
  if (scale_layout == WAVE_MXFP4_SCALE_ROW_MAJOR) {
    // kGroups bytes of each row are contiguous
    if ((ks & 3) == 0) {
      for (int d = threadIdx.x; d < kQuantRows * kGroups / 4; d += 256) {
        const int r = d / (kGroups / 4), gd = d % (kGroups / 4);
        if (row0 + r < rows && g0 + gd * 4 < ks)
          *(uint32_t *)(scale + (int64_t)(row0 + r) * ks + g0 + gd * 4) = tile_scales[d];
      }
    } else {
      for (int b = threadIdx.x; b < kQuantRows * kGroups; b += 256) {
        const int r = b / kGroups, g = b % kGroups;
        if (row0 + r < rows && g0 + g < ks) scale[(int64_t)(row0 + r) * ks + g0 + g] = tile_bytes[b];
      }
    }
  } else {
    // the tile's TC blocks of 256 bytes follow one another (padding rows and groups hold 0)
    const int k_tiles = ksp >> 3;
    uint32_t *out = (uint32_t *)(scale + ((int64_t)row_tile * k_tiles + (int64_t)col_tile * TC) * 256);
    for (int d = threadIdx.x; d < TC * 64; d += 256) {
      if (col_tile * TC + (d >> 6) < k_tiles) out[d] = tile_scales[d];
    }
  }
}

template <int DT, bool GATED>
hipError_t launch_quantize_dt(const QuantParams &p, int num_cus, hipStream_t stream) {
  const int ks = p.k >> 5;
  const int64_t row_tiles = (p.rows + kQuantRows - 1) / kQuantRows;
  // One K tile (256 columns) per workgroup: many small workgroups keep loads and stores of different rows mixed
  // in the memory system (8192 x 8192 bf16: 33.1 us with 8 K tiles per workgroup, 30.7 with 2, 27.9 with 1; the
  // gated form 105.6 / 96.6 / 91.4 us).  Gathered rows run 2 K tiles per workgroup (17.6 / 14.5 / 15.7 us: the row
  // ids are fetched once per workgroup).
  const int64_t narrow = row_tiles * ((ks + 7) / 8), pairs = row_tiles * ((ks + 15) / 16);
  if (narrow > 0x7FFFFFFF) return hipErrorInvalidValue;
  if constexpr (!GATED) {
    if (p.row_ids != nullptr) {
      quantize_kernel<DT, 2, false><<<dim3((unsigned)pairs), 256, 0, stream>>>(p);
      return hipGetLastError();
    }
  }
  (void)num_cus;
  quantize_kernel<DT, 1, GATED><<<dim3((unsigned)narrow), 256, 0, stream>>>(p);
  return hipGetLastError();
}

// Elementwise silu(gate) * up, 8 elements per thread.
template <int DT>
__global__ void __launch_bounds__(256) silu_and_mul_kernel(const uint8_t *__restrict__ gate, const uint8_t *__restrict__ up,
                                                           uint8_t *__restrict__ out, int64_t ld_gate, int64_t ld_up,
                                                           int64_t ld_out, int rows, int n) {
  const int chunks = n >> 3;  // per row
  const int64_t total = (int64_t)rows * chunks;
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t r = i / chunks, c = (i - r * chunks) * 8;
    const v4i g = __builtin_nontemporal_load((const v4i *)(gate + (r * ld_gate + c) * 2));
    const v4i u = __builtin_nontemporal_load((const v4i *)(up + (r * ld_up + c) * 2));
    v4i o;
    o.x = (int)gated_pair<DT>((uint32_t)g.x, (uint32_t)u.x);
    o.y = (int)gated_pair<DT>((uint32_t)g.y, (uint32_t)u.y);
    o.z = (int)gated_pair<DT>((uint32_t)g.z, (uint32_t)u.z);
    o.w = (int)gated_pair<DT>((uint32_t)g.w, (uint32_t)u.w);
    *(v4i *)(out + (r * ld_out + c) * 2) = o;
  }
}

}  // namespace

hipError_t launch_quantize(const void *x, int in_dtype, const int32_t *row_ids, int row_div, int64_t src_rows,
                           uint8_t *q, uint8_t *scale, int64_t rows, int64_t k, int scale_layout, int num_cus,
                           hipStream_t stream) {
  if (rows > 0x7FFFFFFF || k > 0x7FFFFFFF || src_rows > 0x7FFFFFFF) return hipErrorInvalidValue;
  QuantParams p = {};
  p.x = (const uint8_t *)x, p.row_ids = row_ids, p.q = q, p.scale = scale;
  p.ld_x = k, p.rows = (int)rows, p.k = (int)k, p.src_rows = (int)src_rows, p.row_div = row_div > 0 ? row_div : 1;
  p.scale_layout = scale_layout;
  switch (in_dtype) {
    case WAVE_MXFP4_IN_F32: return launch_quantize_dt<WAVE_MXFP4_IN_F32, false>(p, num_cus, stream);
    case WAVE_MXFP4_IN_BF16: return launch_quantize_dt<WAVE_MXFP4_IN_BF16, false>(p, num_cus, stream);
    case WAVE_MXFP4_IN_F16: return launch_quantize_dt<WAVE_MXFP4_IN_F16, false>(p, num_cus, stream);
    default: return hipErrorInvalidValue;
  }
}

hipError_t launch_silu_and_mul_quantize(const void *gate, const void *up, int64_t ld_gate, int64_t ld_up, int in_dtype,
                                        uint8_t *q, uint8_t *scale, int64_t rows, int64_t n, int scale_layout,
                                        int num_cus, hipStream_t stream) {
  if (rows > 0x7FFFFFFF || n > 0x7FFFFFFF) return hipErrorInvalidValue;
  QuantParams p = {};
  p.x = (const uint8_t *)gate, p.up = (const uint8_t *)up, p.q = q, p.scale = scale;
  p.ld_x = ld_gate, p.ld_up = ld_up, p.rows = (int)rows, p.k = (int)n, p.src_rows = (int)rows, p.row_div = 1;
  p.scale_layout = scale_layout;
  switch (in_dtype) {
    case WAVE_MXFP4_IN_BF16: return launch_quantize_dt<WAVE_MXFP4_IN_BF16, true>(p, num_cus, stream);
    case WAVE_MXFP4_IN_F16: return launch_quantize_dt<WAVE_MXFP4_IN_F16, true>(p, num_cus, stream);
    default: return hipErrorInvalidValue;
  }
}

hipError_t launch_silu_and_mul(const void *gate, const void *up, void *out, int64_t ld_gate, int64_t ld_up,
                               int64_t ld_out, int in_dtype, int64_t rows, int64_t n, hipStream_t stream) {
  if (rows > 0x7FFFFFFF || n > 0x7FFFFFFF) return hipErrorInvalidValue;
  const int64_t work = rows * (n >> 3);
  int64_t blocks = (work + 255) / 256;
  if (blocks > 65536) blocks = 65536;
  if (blocks < 1) blocks = 1;
  if (in_dtype == WAVE_MXFP4_IN_BF16)
    silu_and_mul_kernel<WAVE_MXFP4_IN_BF16><<<dim3((unsigned)blocks), 256, 0, stream>>>(
        (const uint8_t *)gate, (const uint8_t *)up, (uint8_t *)out, ld_gate, ld_up, ld_out, (int)rows, (int)n);
  else if (in_dtype == WAVE_MXFP4_IN_F16)
    silu_and_mul_kernel<WAVE_MXFP4_IN_F16><<<dim3((unsigned)blocks), 256, 0, stream>>>(
        (const uint8_t *)gate, (const uint8_t *)up, (uint8_t *)out, ld_gate, ld_up, ld_out, (int)rows, (int)n);
  else
    return hipErrorInvalidValue;
  return hipGetLastError();
}

}  // namespace wave_mxfp4
