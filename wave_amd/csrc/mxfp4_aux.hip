// Small kernels around the GEMM: element decode (bit-exact restatements of the
// reference's mxfp4_to_f32 / e8m0_to_f32, wave_lang/kernel/wave/utils/
// mxfp_utils.py:60-95), dequantisation, the two layout shuffles
// (mxfp_utils.py:98-128), the split-K reduction and a one-thread-per-element
// GEMM used to cross-check the MFMA kernels on the device.
#include "mxfp4_common.h"
#include "mxfp4_group_table.h"

namespace wave_mxfp4 {

constexpr int kThreads = 256;

static inline unsigned blocks_for(int64_t work, int per_block) {
  int64_t b = (work + per_block - 1) / per_block;
  if (b < 1) b = 1;
  if (b > 1048576) b = 1048576;
  return (unsigned)b;
}

// ---- packed e2m1 -> f32, one thread per packed byte (grid-stride) ----
__global__ void to_f32_kernel(const uint8_t *__restrict__ q, float *__restrict__ out, int64_t nbytes) {
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < nbytes;
       i += (int64_t)gridDim.x * blockDim.x) {
    const uint32_t b = q[i];
    v2f v = {e2m1_to_f32(b & 0xFu), e2m1_to_f32(b >> 4)};
    *(v2f *)(out + 2 * i) = v;
  }
}

__global__ void e8m0_kernel(const uint8_t *__restrict__ s, float *__restrict__ out, int64_t count) {
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < count;
       i += (int64_t)gridDim.x * blockDim.x)
    out[i] = e8m0_to_f32(s[i]);
}

// out[r, e] = value * scale(r, e/32); one thread per packed byte.
__global__ void dequant_kernel(const uint8_t *__restrict__ q, const uint8_t *__restrict__ scale,
                               float *__restrict__ out, int64_t rows, int64_t kp, int64_t ks, int64_t ksp,
                               int layout) {
  const int64_t nbytes = rows * kp;
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < nbytes;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t r = i / kp, kb = i - r * kp, g = kb >> 4;
    const uint32_t sbyte = scale[scale_offset(layout, r, g, ks, ksp)];
    const float sc = e8m0_to_f32(sbyte);
    const uint32_t b = q[i];
    v2f v = {e2m1_to_f32(b & 0xFu) * sc, e2m1_to_f32(b >> 4) * sc};
    *(v2f *)(out + 2 * i) = v;
  }
}

// One thread per byte of the padded, tile-ordered output.
__global__ void e8m0_shuffle_kernel(const uint8_t *__restrict__ scale, uint8_t *__restrict__ out,
                                    int64_t rows, int64_t ks, int64_t rows_p, int64_t ksp) {
  const int64_t total = rows_p * ksp;
  for (int64_t o = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; o < total;
       o += (int64_t)gridDim.x * blockDim.x) {
    // invert the offset formula: o = rt*(ksp/8*256) + kt*256 + g4*64 + r16*4 + kh*2 + rh
    const int64_t tile_row_bytes = (ksp >> 3) * 256;
    const int64_t rt = o / tile_row_bytes;
    const int64_t w = o - rt * tile_row_bytes;
    const int64_t kt = w >> 8, in = w & 255;
    const int64_t g4 = in >> 6, r16 = (in >> 2) & 15, kh = (in >> 1) & 1, rh = in & 1;
    const int64_t r = rt * 32 + rh * 16 + r16;
    const int64_t g = kt * 8 + kh * 4 + g4;
    out[o] = (r < rows && g < ks) ? scale[r * ks + g] : (uint8_t)0;
  }
}

// Any scale layout -> any scale layout, one thread per dword of the padded
// (32 rows x 8 groups) index space; every destination byte, padding included, is
// written exactly once.
__global__ void scale_convert_kernel(const uint8_t *__restrict__ src, int src_layout, uint8_t *__restrict__ dst,
                                     int dst_layout, int64_t rows, int64_t ks, int64_t rows_p, int64_t ksp) {
  const int64_t total = rows_p * (ksp >> 2);
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < total;
       i += (int64_t)gridDim.x * blockDim.x) {
    // consecutive threads walk the MFMA32 order: block (row tile, K tile), lane, so
    // that the writes of the common conversion (to MFMA32) are whole dwords
    const int64_t blk = i >> 6, lane = i & 63;
    const int64_t k_tiles = ksp >> 3;
    const int64_t rt = blk / k_tiles, kt = blk - rt * k_tiles;
    const int64_t r = rt * 32 + (lane & 31), fg = lane >> 5;
    uint32_t word = 0;
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const int64_t g = kt * 8 + 2 * t + fg;
      const uint32_t b = (r < rows && g < ks) ? src[scale_offset(src_layout, r, g, ks, ksp)] : 0u;
      word |= b << (8 * t);
    }
    if (dst_layout == WAVE_MXFP4_SCALE_MFMA32) {
      *(uint32_t *)(dst + i * 4) = word;
    } else {
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const int64_t g = kt * 8 + 2 * t + fg;
        if (dst_layout == WAVE_MXFP4_SCALE_ROW_MAJOR) {
          if (r < rows && g < ks) dst[r * ks + g] = (uint8_t)(word >> (8 * t));
        } else {
          dst[scale_offset(dst_layout, r, g, ks, ksp)] = (uint8_t)(word >> (8 * t));
        }
      }
    }
  }
}

// Row-major -> MFMA32, the conversion in front of every tile GEMM with row-major scales (8-byte reads as two
// dwords where the rows start on dwords, ks % 4 == 0; byte reads otherwise).  A workgroup takes 32 blocks of (32 rows x one K
// tile): 32 rows x 32 K tiles, or for short rows 64 x 16 or 128 x 8, so that all
// of its threads have a piece whatever K is (with 16 K tiles a row, K = 4096, half
// of them had none).  8-byte reads that walk each row contiguously, the even and
// odd groups of a K tile split with v_perm into the two dwords of its block (lanes
// r%32 and 32 + r%32), a pass through LDS (block stride 65 dwords), and dword
// writes that walk the destination contiguously.
// blockIdx.z picks one of two tensors with the same ks (the A and B scales of a
// GEMM go through one launch; rows of one of them 0 for a single tensor).
// With gt.table the launch's first workgroup builds the M tile table of a grouped
// GEMM before its share of the scales (mxfp4_group_table.h): the table only needs
// the offsets, so it costs the call no launch of its own.
// K tiles of a row that one workgroup walks, as a power of two: 5, 4 or 3.
__host__ __device__ inline int scale_wg_kt_log(int k_tiles) { return k_tiles > 16 ? 5 : k_tiles > 8 ? 4 : 3; }
__global__ void __launch_bounds__(256) scale_to_mfma32_kernel(const uint8_t *__restrict__ src0,
                                                              uint8_t *__restrict__ dst0, int rows0,
                                                              const uint8_t *__restrict__ src1,
                                                              uint8_t *__restrict__ dst1, int rows1, int ks,
                                                              const GroupTableArgs gt) {
  __shared__ uint32_t stage[32 * 65];
  if (gt.table != nullptr && blockIdx.x == 0 && blockIdx.y == 0 && blockIdx.z == 0) {
    __shared__ int wave_sums[4];
    __shared__ int carry[2];
    build_group_tile_table<256>(gt, wave_sums, carry);
  }
  const uint8_t *src = blockIdx.z ? src1 : src0;
  uint8_t *dst = blockIdx.z ? dst1 : dst0;
  const int rows = blockIdx.z ? rows1 : rows0;
  const int k_tiles = (ks + 7) >> 3;  // the last K tile may hold fewer than 8 groups (the rest is written as 0)
  const int kt_log = scale_wg_kt_log(k_tiles), kt_mask = (1 << kt_log) - 1;
  const int rt0 = blockIdx.x << (5 - kt_log), kt0 = blockIdx.y << kt_log;  // row tiles along x: up to 2^31 - 1 workgroups
  const int row_base = rt0 * 32;
  if (row_base >= rows) return;  // the grid is sized for the taller tensor
  const int t = threadIdx.x;
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const int unit = t + 256 * u, r = unit >> kt_log, ktl = unit & kt_mask;
    const int row = row_base + r, kt = kt0 + ktl;
    uint2 v = make_uint2(0u, 0u);
    if (row < rows && kt < k_tiles) {
      const uint8_t *at = src + (int64_t)row * ks + (int64_t)kt * 8;
      if ((ks & 3) == 0) {
        v.x = *(const uint32_t *)at;
        if (kt * 8 + 4 < ks) v.y = *(const uint32_t *)(at + 4);
      } else {
        // rows that do not start on dwords (K % 128 != 0): byte by byte, groups past the end of the row stay 0
        const int valid = min(8, ks - kt * 8);
        for (int b = 0; b < valid; ++b) {
          const uint32_t byte = at[b];
          if (b < 4) v.x |= byte << (8 * b); else v.y |= byte << (8 * (b - 4));
        }
      }
    }
    const int blk = ((r >> 5) << kt_log) + ktl;
    stage[blk * 65 + (r & 31)] = __builtin_amdgcn_perm(v.y, v.x, 0x06040200u);       // groups 0, 2, 4, 6
    stage[blk * 65 + 32 + (r & 31)] = __builtin_amdgcn_perm(v.y, v.x, 0x07050301u);  // groups 1, 3, 5, 7
  }
  __syncthreads();
  uint32_t *out = (uint32_t *)dst;
#pragma unroll
  for (int u = 0; u < 8; ++u) {
    const int d = t + 256 * u, blk = d >> 6, lane = d & 63;
    const int rt = rt0 + (blk >> kt_log), kt = kt0 + (blk & kt_mask);
    if (kt < k_tiles && rt * 32 < rows) out[((int64_t)rt * k_tiles + kt) * 64 + lane] = stage[blk * 65 + lane];
  }
}

// e8m0_shuffle -> MFMA32: both keep one 256-byte block per (32 rows, K tile) in the same block order, so the
// conversion permutes bytes inside a block.  One thread per destination dword (lane (g%2)*32 + r%32, bytes
// t = 0..3 = groups 2t + g%2): its bytes come from the two source dwords (g%4)*16 + r%16 for g%4 = g%2 and
// 2 + g%2, byte (g/4)*2 + (r%32)/16 of each.  blockIdx.y picks one of two tensors.
__global__ void __launch_bounds__(256) scale_shuffle_to_mfma32_kernel(const uint32_t *__restrict__ src0,
                                                                      uint32_t *__restrict__ dst0, int64_t dwords0,
                                                                      const uint32_t *__restrict__ src1,
                                                                      uint32_t *__restrict__ dst1, int64_t dwords1) {
  const uint32_t *src = blockIdx.y ? src1 : src0;
  uint32_t *dst = blockIdx.y ? dst1 : dst0;
  const int64_t dwords = blockIdx.y ? dwords1 : dwords0;
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < dwords; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t blk = i >> 6;
    const int lane = (int)(i & 63), r32 = lane & 31, gpar = lane >> 5;
    const uint32_t d0 = src[blk * 64 + gpar * 16 + (r32 & 15)], d1 = src[blk * 64 + (2 + gpar) * 16 + (r32 & 15)];
    dst[i] = __builtin_amdgcn_perm(d1, d0, (r32 >> 4) ? 0x07030501u : 0x06020400u);
  }
}

// dst[r, g] = src[r]: one scale per row spread over the row's ks groups.
__global__ void scale_spread_rows_kernel(const uint8_t *__restrict__ src, uint8_t *__restrict__ dst, int64_t rows,
                                         int64_t ks) {
  const int64_t total = rows * ks;
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x)
    dst[i] = src[i / ks];
}

// One thread per 16-byte chunk.
__global__ void b_preshuffle_kernel(const uint8_t *__restrict__ b, uint8_t *__restrict__ out, int64_t rows,
                                    int64_t kp) {
  const int64_t chunks_per_row = kp >> 4;
  const int64_t total = rows * chunks_per_row;
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < total;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t n = i / chunks_per_row, c = i - n * chunks_per_row;
    const v4i v = *(const v4i *)(b + n * kp + c * 16);
    *(v4i *)(out + b_preshuffle_offset(n, c * 16, kp)) = v;
  }
}

// 8-bit B [rows, k] -> the order the B-direct MXFP8 kernel reads (mxfp8_gemm_asym.hip): blocks of 32 rows x 128
// bytes, block (n / 32, kt) at ((n / 32) * (k / 128) + kt) * 4096, its 16-byte pieces as [K step][half][lane],
// lane = 32 * g + r holding row r's bytes 64 * step + 32 * half + 16 * g .. + 15.  One thread per piece of the result.
__global__ void b8_preshuffle_kernel(const uint8_t *__restrict__ b, uint8_t *__restrict__ out, int64_t rows, int64_t k) {
  const int64_t total = rows * (k >> 4), k_tiles = k >> 7;
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t blk = i >> 8, nb = blk / k_tiles, kt = blk - nb * k_tiles;
    const int piece = (int)(i & 255), q = piece >> 6, lane = piece & 63;
    const int64_t row = nb * 32 + (lane & 31);
    const int64_t col = kt * 128 + (q >> 1) * 64 + (q & 1) * 32 + (lane >> 5) * 16;
    *(v4i *)(out + i * 16) = *(const v4i *)(b + row * k + col);
  }
}

// Rows of a [2 * half_rows, row_bytes] matrix whose first half is a gate projection and whose second half the
// matching up projection, interleaved in blocks of `block` rows: out block 2 b = gate rows block b, out block
// 2 b + 1 = up rows block b.  One thread per 4 bytes (row_bytes % 4 == 0) or per byte.
template <typename T>
__global__ void interleave_rows_kernel(const T *__restrict__ src, T *__restrict__ dst, int64_t half_rows, int64_t row_units,
                                       int block) {
  const int64_t total = 2 * half_rows * row_units;
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t r = i / row_units, c = i - r * row_units;
    const int64_t blk = r / block, in = r - blk * block;
    const int64_t from = (blk & 1 ? half_rows : 0) + (blk >> 1) * block + in;
    dst[i] = src[from * row_units + c];
  }
}

// C = sum over splits of partial[s], converted to the output type.  Fixed
// summation order, so the result does not depend on scheduling.
__global__ void splitk_reduce_kernel(const float *__restrict__ partial, void *__restrict__ c, int64_t mn,
                                     int splits, int out_bf16) {
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < mn;
       i += (int64_t)gridDim.x * blockDim.x) {
    float acc = partial[i];
    for (int s = 1; s < splits; ++s) acc += partial[(int64_t)s * mn + i];
    if (out_bf16)
      ((__bf16 *)c)[i] = (__bf16)acc;
    else
      ((float *)c)[i] = acc;
  }
}

// The same, four consecutive elements per thread (16-byte loads of every split in flight together, one 8- or
// 16-byte store); mn % 4 == 0, c 16-byte aligned.  SPLITS > 0 fixes the count at compile time.
template <int SPLITS, bool OUT_BF16>
__global__ void __launch_bounds__(256) splitk_reduce4_kernel(const float *__restrict__ partial, void *__restrict__ c,
                                                             int64_t mn4, int splits_rt) {
  const int splits = SPLITS > 0 ? SPLITS : splits_rt;
  const v4f *src = (const v4f *)partial;
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < mn4; i += (int64_t)gridDim.x * blockDim.x) {
    v4f acc;
    if constexpr (SPLITS > 0) {
      v4f part[SPLITS];
#pragma unroll
      for (int s = 0; s < SPLITS; ++s) part[s] = __builtin_nontemporal_load(src + (int64_t)s * mn4 + i);
      acc = part[0];
#pragma unroll
      for (int s = 1; s < SPLITS; ++s) acc += part[s];  // the order of the one-element kernel
    } else {
      acc = __builtin_nontemporal_load(src + i);
      for (int s = 1; s < splits; ++s) acc += __builtin_nontemporal_load(src + (int64_t)s * mn4 + i);
    }
    if constexpr (OUT_BF16) {
      typedef __bf16 bf4 __attribute__((ext_vector_type(4)));
      bf4 o;
#pragma unroll
      for (int e = 0; e < 4; ++e) o[e] = (__bf16)acc[e];
      ((bf4 *)c)[i] = o;
    } else {
      ((v4f *)c)[i] = acc;
    }
  }
}

// One thread per C element: table decode, f32 multiply-add in K order.  Slow;
// exists so the MFMA kernels can be checked on the device at any shape.
__global__ void naive_gemm_kernel(const GemmParams p) {
  const int64_t total = (int64_t)p.m * p.n;
  for (int64_t idx = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; idx < total;
       idx += (int64_t)gridDim.x * blockDim.x) {
    const int m = (int)(idx / p.n), n = (int)(idx - (int64_t)m * p.n);
    const uint8_t *bp = p.b;
    const uint8_t *bsp = p.b_scale;
    if (p.num_groups > 0) {
      int e = 0;
      while (e < p.num_groups && !(m >= p.offsets[e] && m < p.offsets[e + 1])) ++e;
      if (e == p.num_groups) continue;  // row belongs to no group: left untouched
      bp += (int64_t)e * p.b_group_stride;
      bsp += (int64_t)e * p.b_scale_group_stride;
    }
    float acc = 0.f;
    for (int g = 0; g < p.ks; ++g) {
      const uint32_t sa = p.a_scale[scale_offset(p.a_scale_layout, m, g, p.ks, p.ksp)];
      const uint32_t sb = bsp[scale_offset(p.b_scale_layout, n, g, p.ks, p.ksp)];
      const float fa = e8m0_to_f32(sa), fb = e8m0_to_f32(sb);
      // one scale group = 16 packed bytes, contiguous in both B layouts
      const v4i av = *(const v4i *)(p.a + (int64_t)m * p.kp + g * 16);
      const v4i bv = *(const v4i *)(p.b_preshuffled ? bp + b_preshuffle_offset(n, g * 16, p.kp)
                                                    : bp + (int64_t)n * p.kp + g * 16);
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        const uint32_t aw = (uint32_t)av[w], bw = (uint32_t)bv[w];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const uint32_t ac = (aw >> (4 * j)) & 0xFu, bc = (bw >> (4 * j)) & 0xFu;
          acc += (e2m1_to_f32(ac) * fa) * (e2m1_to_f32(bc) * fb);
        }
      }
    }
    if (p.out_bf16)
      ((__bf16 *)p.c)[idx] = (__bf16)acc;
    else
      ((float *)p.c)[idx] = acc;
  }
}

hipError_t launch_to_f32(const uint8_t *q, float *out, int64_t rows, int64_t kp, hipStream_t stream) {
  const int64_t n = rows * kp;
  if (n == 0) return hipSuccess;
  to_f32_kernel<<<blocks_for(n, kThreads), kThreads, 0, stream>>>(q, out, n);
  return hipGetLastError();
}

hipError_t launch_e8m0_to_f32(const uint8_t *s, float *out, int64_t count, hipStream_t stream) {
  if (count == 0) return hipSuccess;
  e8m0_kernel<<<blocks_for(count, kThreads), kThreads, 0, stream>>>(s, out, count);
  return hipGetLastError();
}

hipError_t launch_dequant(const uint8_t *q, const uint8_t *scale, float *out, int64_t rows, int64_t k,
                          int layout, hipStream_t stream) {
  const int64_t n = rows * (k / 2);
  if (n == 0) return hipSuccess;
  const int64_t ks = k / 32, ksp = (ks + 7) / 8 * 8;
  dequant_kernel<<<blocks_for(n, kThreads), kThreads, 0, stream>>>(q, scale, out, rows, k / 2, ks, ksp,
                                                                  layout);
  return hipGetLastError();
}

hipError_t launch_e8m0_shuffle(const uint8_t *scale, uint8_t *out, int64_t rows, int64_t ks,
                               hipStream_t stream) {
  const int64_t rows_p = (rows + 31) / 32 * 32, ksp = (ks + 7) / 8 * 8;
  const int64_t n = rows_p * ksp;
  if (n == 0) return hipSuccess;
  e8m0_shuffle_kernel<<<blocks_for(n, kThreads), kThreads, 0, stream>>>(scale, out, rows, ks, rows_p, ksp);
  return hipGetLastError();
}

hipError_t launch_scale_convert(const uint8_t *src, int src_layout, uint8_t *dst, int dst_layout, int64_t rows,
                                int64_t ks, hipStream_t stream) {
  const int64_t rows_p = (rows + 31) / 32 * 32, ksp = (ks + 7) / 8 * 8;
  const int64_t n = rows_p * (ksp / 4);
  if (n == 0) return hipSuccess;
  if (src_layout == WAVE_MXFP4_SCALE_ROW_MAJOR && dst_layout == WAVE_MXFP4_SCALE_MFMA32 && (ks & 3) == 0 &&
      ((uintptr_t)src & 3) == 0 && rows < ((int64_t)1 << 31) && (ksp / 8 + 31) / 32 <= 65535) {
    const int kt_log = scale_wg_kt_log((int)(ksp / 8));
    const int64_t rows_wg = 1024 >> kt_log, per_wg = (int64_t)1 << kt_log;  // rows and K tiles a workgroup takes
    dim3 grid((unsigned)((rows + rows_wg - 1) / rows_wg), (unsigned)((ksp / 8 + per_wg - 1) / per_wg), 1);
    scale_to_mfma32_kernel<<<grid, 256, 0, stream>>>(src, dst, (int)rows, nullptr, nullptr, 0, (int)ks, GroupTableArgs{});
    return hipGetLastError();
  }
  if (src_layout == WAVE_MXFP4_SCALE_E8M0_SHUFFLE && dst_layout == WAVE_MXFP4_SCALE_MFMA32 && ((uintptr_t)src & 3) == 0) {
    scale_shuffle_to_mfma32_kernel<<<dim3(blocks_for(n, kThreads), 1), kThreads, 0, stream>>>(
        (const uint32_t *)src, (uint32_t *)dst, n, nullptr, nullptr, 0);
    return hipGetLastError();
  }
  scale_convert_kernel<<<blocks_for(n, kThreads), kThreads, 0, stream>>>(src, src_layout, dst, dst_layout, rows,
                                                                        ks, rows_p, ksp);
  return hipGetLastError();
}

// e8m0_shuffle -> MFMA32 for the scales of both GEMM operands in one launch.
hipError_t launch_scale_pair_shuffle_to_mfma32(const uint8_t *a_src, uint8_t *a_dst, int64_t a_rows, const uint8_t *b_src,
                                               uint8_t *b_dst, int64_t b_rows, int64_t ks, hipStream_t stream) {
  if ((((uintptr_t)a_src | (uintptr_t)b_src) & 3) != 0) return hipErrorInvalidValue;
  const int64_t ksp = (ks + 7) / 8 * 8;
  const int64_t na = (a_rows + 31) / 32 * 32 * (ksp / 4), nb = (b_rows + 31) / 32 * 32 * (ksp / 4);
  scale_shuffle_to_mfma32_kernel<<<dim3(blocks_for(na > nb ? na : nb, kThreads), 2), kThreads, 0, stream>>>(
      (const uint32_t *)a_src, (uint32_t *)a_dst, na, (const uint32_t *)b_src, (uint32_t *)b_dst, nb);
  return hipGetLastError();
}

// Row-major -> MFMA32 for the scales of both GEMM operands in one launch.
// Returns hipErrorInvalidValue (nothing launched) when the fast kernel does not apply.
// With `table` the launch's first workgroup also builds the M tile table of a grouped GEMM, see the kernel.
// One of a_rows, b_rows may be 0: the other tensor alone.
hipError_t launch_scale_pair_to_mfma32(const uint8_t *a_src, uint8_t *a_dst, int64_t a_rows, const uint8_t *b_src,
                                       uint8_t *b_dst, int64_t b_rows, int64_t ks, hipStream_t stream,
                                       const GroupTableArgs *table) {
  if (a_rows == 0 && b_rows > 0) {  // B alone: as the launch's first tensor
    a_src = b_src, a_dst = b_dst, a_rows = b_rows;
    b_rows = 0;
  }
  const int64_t rows_max = a_rows > b_rows ? a_rows : b_rows;
  // (dword reads where the rows start on dwords, byte reads otherwise)
  const bool dwords = (ks & 3) == 0;
  if (ks == 0 || (dwords && (((uintptr_t)a_src & 3) != 0 || (b_rows > 0 && ((uintptr_t)b_src & 3) != 0))) ||
      rows_max >= ((int64_t)1 << 31) || ((ks + 7) / 8 + 31) / 32 > 65535 || a_rows <= 0 || b_rows < 0)
    return hipErrorInvalidValue;
  const int kt_log = scale_wg_kt_log((int)((ks + 7) / 8));
  const int64_t rows_wg = 1024 >> kt_log;  // rows a workgroup takes
  const int64_t k_tiles = (ks + 7) / 8, per_wg = (int64_t)1 << kt_log;
  dim3 grid((unsigned)((rows_max + rows_wg - 1) / rows_wg), (unsigned)((k_tiles + per_wg - 1) / per_wg), b_rows > 0 ? 2 : 1);
  scale_to_mfma32_kernel<<<grid, 256, 0, stream>>>(a_src, a_dst, (int)a_rows, b_src, b_dst, (int)b_rows, (int)ks,
                                                   table ? *table : GroupTableArgs{});
  return hipGetLastError();
}

hipError_t launch_scale_spread_rows(const uint8_t *src, uint8_t *dst, int64_t rows, int64_t ks, hipStream_t stream) {
  scale_spread_rows_kernel<<<blocks_for(rows * ks, 256), 256, 0, stream>>>(src, dst, rows, ks);
  return hipGetLastError();
}

hipError_t launch_b8_preshuffle(const uint8_t *b, uint8_t *out, int64_t rows, int64_t k, hipStream_t stream) {
  const int64_t n = rows * (k / 16);
  if (n == 0) return hipSuccess;
  b8_preshuffle_kernel<<<blocks_for(n, kThreads), kThreads, 0, stream>>>(b, out, rows, k);
  return hipGetLastError();
}

hipError_t launch_b_preshuffle(const uint8_t *b, uint8_t *out, int64_t rows, int64_t kp,
                               hipStream_t stream) {
  const int64_t n = rows * (kp / 16);
  if (n == 0) return hipSuccess;
  b_preshuffle_kernel<<<blocks_for(n, kThreads), kThreads, 0, stream>>>(b, out, rows, kp);
  return hipGetLastError();
}

hipError_t launch_interleave_rows(const uint8_t *src, uint8_t *dst, int64_t half_rows, int64_t row_bytes, int block,
                                  hipStream_t stream) {
  const int64_t n = 2 * half_rows * row_bytes;
  if (n == 0) return hipSuccess;
  if (row_bytes % 4 == 0 && ((uintptr_t)src & 3) == 0 && ((uintptr_t)dst & 3) == 0)
    interleave_rows_kernel<uint32_t><<<blocks_for(n / 4, kThreads), kThreads, 0, stream>>>(
        (const uint32_t *)src, (uint32_t *)dst, half_rows, row_bytes / 4, block);
  else
    interleave_rows_kernel<uint8_t><<<blocks_for(n, kThreads), kThreads, 0, stream>>>(src, dst, half_rows, row_bytes, block);
  return hipGetLastError();
}

hipError_t launch_splitk_reduce(const float *partial, void *c, int64_t mn, int splits, int out_bf16,
                                hipStream_t stream) {
  if (mn == 0) return hipSuccess;
  if (mn % 4 == 0 && ((uintptr_t)c & 15) == 0 && ((uintptr_t)partial & 15) == 0) {
    const int64_t mn4 = mn / 4;
    const unsigned grid = blocks_for(mn4, kThreads);
#define WAVE_REDUCE4(S)                                                                                    \
  (out_bf16 ? splitk_reduce4_kernel<S, true><<<grid, kThreads, 0, stream>>>(partial, c, mn4, splits)       \
            : splitk_reduce4_kernel<S, false><<<grid, kThreads, 0, stream>>>(partial, c, mn4, splits))
    switch (splits) {
      case 2: WAVE_REDUCE4(2); break;
      case 3: WAVE_REDUCE4(3); break;
      case 4: WAVE_REDUCE4(4); break;
      case 5: WAVE_REDUCE4(5); break;
      case 6: WAVE_REDUCE4(6); break;
      case 7: WAVE_REDUCE4(7); break;
      case 8: WAVE_REDUCE4(8); break;
      default: WAVE_REDUCE4(0); break;
    }
#undef WAVE_REDUCE4
    return hipGetLastError();
  }
  splitk_reduce_kernel<<<blocks_for(mn, kThreads), kThreads, 0, stream>>>(partial, c, mn, splits, out_bf16);
  return hipGetLastError();
}

hipError_t launch_naive_gemm(const GemmParams &p, hipStream_t stream) {
  const int64_t n = (int64_t)p.m * p.n;
  if (n == 0) return hipSuccess;
  naive_gemm_kernel<<<blocks_for(n, kThreads), kThreads, 0, stream>>>(p);
  return hipGetLastError();
}

}  // namespace wave_mxfp4
